// Unary functions of a 16-bit dtype by table.
//
// A unary op on bf16 or f16 has 65536 possible inputs.  For the ops whose evaluation is long (the bit-exact libm
// restatements of mathfn.hpp cost 60 to 170 instructions per element, which makes tanh_bf16 on [8192,8192] an
// ALU-bound 210 us kernel where the bytes would take 45 us), the library keeps, per op, dtype and device, a table of
// all 65536 results - built once by running the op's own elementwise kernel over the 65536 input codes, so a table
// entry IS the bits that kernel produces.  A large contiguous call then runs lut16_kernel: one 1024-thread block per CU
// copies the 128 KB table into LDS (gfx950 has 160 KB per CU) and streams its share of the input through it, eight
// elements per 16-byte vector, one LDS read per element.  A transposed view whose tiles can move as 16-byte vectors has
// the same arrangement with a tile next to the table (ew_trvp_kernel); other layouts go through the ordinary strided
// kernels with a functor that reads the table from global memory, where the few KB that real data touch stay in the
// vector cache.  Small calls, and calls while a graph capture is open and the table does not exist yet (building
// it allocates), keep the arithmetic path.
#pragma once
#include <algorithm>

#include "elementwise.hpp"

namespace mxh {

constexpr int LUT_BLOCK = 1024;
constexpr size_t LUT_BYTES = 65536 * sizeof(uint16_t);
constexpr size_t LUT_MIN_ELEMS = 1u << 20;        // below this the table's 128 KB per block are not worth copying

bool capture_open();      // runtime.hip: a graph capture is being recorded

typedef uint32_t lut_u4 __attribute__((ext_vector_type(4)));

static __global__ __launch_bounds__(256) void lut16_iota_kernel(uint16_t* codes) {
    codes[blockIdx.x * 256 + threadIdx.x] = (uint16_t)(blockIdx.x * 256 + threadIdx.x);
}

template <bool STREAM>
__global__ __launch_bounds__(LUT_BLOCK) void lut16_kernel(const uint16_t* __restrict__ table, const uint16_t* in, uint16_t* out, size_t n) {
    extern __shared__ __attribute__((aligned(16))) uint16_t lut[];
    for (int i = threadIdx.x; i < (int)(LUT_BYTES / 16); i += LUT_BLOCK) ((lut_u4*)lut)[i] = ((const lut_u4*)table)[i];
    __syncthreads();
    const size_t nvec = n / 8;
    const lut_u4* vin = (const lut_u4*)in;
    lut_u4* vout = (lut_u4*)out;
    constexpr int U = 2;                              // vectors in flight per thread
    const size_t stride = (size_t)gridDim.x * LUT_BLOCK * U;
    for (size_t v0 = (size_t)blockIdx.x * LUT_BLOCK * U + threadIdx.x; v0 < nvec; v0 += stride) {
        lut_u4 x[U];
#pragma unroll
        for (int k = 0; k < U; ++k)
            if (v0 + (size_t)k * LUT_BLOCK < nvec) x[k] = ld_vec<STREAM>(vin + v0 + (size_t)k * LUT_BLOCK);
#pragma unroll
        for (int k = 0; k < U; ++k) {
            if (v0 + (size_t)k * LUT_BLOCK >= nvec) break;
            lut_u4 r;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const uint32_t w = x[k][e];
                r[e] = (uint32_t)lut[w & 0xFFFFu] | ((uint32_t)lut[w >> 16] << 16);
            }
            st_vec<STREAM>(vout + v0 + (size_t)k * LUT_BLOCK, r);
        }
    }
    const size_t tail = n - nvec * 8;                 // fewer than eight elements after the last whole vector
    if (blockIdx.x == 0 && threadIdx.x < tail) out[nvec * 8 + threadIdx.x] = lut[in[nvec * 8 + threadIdx.x]];
}

// The table read from global memory, as a functor of the strided kernels.
template <class T>
struct OpLut16 {
    using In = T;
    using Out = T;
    static constexpr int NIN = 1;
    const uint16_t* table;
    __device__ T operator()(T x) const {
        T r;
        r.bits = table[x.bits];
        return r;
    }
};


// The table functor inside the persistent transposing kernel (ew_trvp_kernel): the table sits in LDS in front of the tile.
template <class T>
struct TrvDeviceOp<OpLut16<T>> {
    static constexpr size_t PREFIX = LUT_BYTES;
    const uint16_t* lut;
    // every thread of the block takes part; the caller's barrier follows
    __device__ TrvDeviceOp(const OpLut16<T>& op, void* smem) : lut((const uint16_t*)smem) {
        for (int i = threadIdx.x; i < (int)(LUT_BYTES / 16); i += blockDim.x) ((lut_u4*)smem)[i] = ((const lut_u4*)op.table)[i];
    }
    __device__ T operator()(T x) const {
        T r;
        r.bits = lut[x.bits];
        return r;
    }
};

// Device pointer to the table of Op on the current device; built on first use.  Null when it cannot be built now.
template <class Op>
const uint16_t* lut16_table() {
    static uint16_t* tables[16] = {nullptr};          // one per device; the entry points hold the library's lock
    static_assert(sizeof(typename Op::In) == 2 && sizeof(typename Op::Out) == 2, "tables are for 16-bit dtypes");
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return nullptr;
    if (tables[dev]) return tables[dev];
    if (capture_open()) return nullptr;               // building allocates and synchronises
    uint16_t *codes = nullptr, *tab = nullptr;
    if (hipMalloc((void**)&codes, LUT_BYTES) != hipSuccess) return nullptr;
    if (hipMalloc((void**)&tab, LUT_BYTES) != hipSuccess) { (void)hipFree(codes); return nullptr; }
    hipLaunchKernelGGL(lut16_iota_kernel, dim3(256), dim3(256), 0, stream(), codes);
    MXH_LAUNCH_CHECK("lut16_iota");
    ew_unary(65536, 1, nullptr, codes, tab, Op{});    // the op's own kernel: the table holds exactly its bits
    hipError_t e = hipStreamSynchronize(stream());
    (void)hipFree(codes);
    if (e != hipSuccess) { (void)hipFree(tab); set_status(ERR_LAUNCH, "building a 16-bit function table", (int)e); return nullptr; }
    tables[dev] = tab;                                // kept until the process ends
    return tab;
}

// hip_<op>_<bf16|f16> through the table.  False: not applicable here, the caller runs the arithmetic kernel.
template <class Op>
bool lut16_unary(size_t num_els, size_t num_dims, const size_t* md, const void* input, void* out) {
    using T = typename Op::In;
    if (num_els < LUT_MIN_ELEMS || !out) return false;
    if (md && num_dims > 64) return false;
    const uint16_t* table = lut16_table<Op>();
    if (!table) return false;
    const size_t off = md ? md[2 * num_dims] : 0;
    const T* src = input ? (const T*)input + off : (const T*)out;
    const bool contiguous = !input || !md || ref_is_contiguous(num_dims, md, md + num_dims);
    if (contiguous && (uintptr_t)src % 16 == 0 && (uintptr_t)out % 16 == 0) {
        static bool attr_set[16][2] = {{false}};
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return false;
        const int ncu = device_cus(dev);
        if (!ncu) return false;
        const bool streams = ew_stream_bytes() != 0 && num_els * 4 >= ew_stream_bytes();
        if (!attr_set[dev][streams]) {
            hipError_t e = streams ? hipFuncSetAttribute((const void*)lut16_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)LUT_BYTES)
                                   : hipFuncSetAttribute((const void*)lut16_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)LUT_BYTES);
            if (e != hipSuccess) { (void)hipGetLastError(); return false; }
            attr_set[dev][streams] = true;
        }
        const size_t nvec = num_els / 8;
        const unsigned blocks = (unsigned)std::min<size_t>((size_t)ncu, cdiv(nvec, (size_t)LUT_BLOCK * 2));
        if (streams)
            hipLaunchKernelGGL(lut16_kernel<true>, dim3(blocks), dim3(LUT_BLOCK), LUT_BYTES, stream(), table, (const uint16_t*)src, (uint16_t*)out, num_els);
        else
            hipLaunchKernelGGL(lut16_kernel<false>, dim3(blocks), dim3(LUT_BLOCK), LUT_BYTES, stream(), table, (const uint16_t*)src, (uint16_t*)out, num_els);
        MXH_LAUNCH_CHECK("lut16");
        return true;
    }
    ew_unary(num_els, num_dims, md, input, out, OpLut16<T>{table});
    return true;
}

}  // namespace mxh
