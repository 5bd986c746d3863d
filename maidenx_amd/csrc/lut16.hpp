// Unary functions of a 16-bit dtype by table.
//
// A unary op on bf16 or f16 has 65536 possible inputs.  For the ops whose evaluation is long (the bit-exact libm
// restatements of mathfn.hpp cost 60 to 170 instructions per element, which makes tanh_bf16 on [8192,8192] an
// ALU-bound 210 us kernel where the bytes would take 45 us), the library keeps, per op, dtype and device, a table of
// all 65536 results - built once by running the op's own elementwise kernel over the 65536 input codes, so a table
// entry IS the bits that kernel produces.  A large contiguous call then runs lut16_kernel: one 1024-thread block per CU
// copies the 128 KB table into LDS (gfx950 has 160 KB per CU) and streams its share of the input through it, eight
// elements per 16-byte vector, one LDS read per element.  A transposed view whose tiles can move as 16-byte vectors has
// the same arrangement with a tile next to the table (lut16_trv_kernel); other layouts go through the ordinary strided
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

inline int lut16_cus(int dev) {
    static int cus[16] = {0};
    if (dev < 0 || dev >= 16) return 0;
    if (!cus[dev]) {
        hipDeviceProp_t prop;
        if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return 0;
        cus[dev] = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    }
    return cus[dev];
}

// A transposed view through the table: ew_trv_kernel's tiles (256 bytes of the input's unit-stride dim by 64 of the
// output's), worked through by one persistent 1024-thread block per CU that holds the table in LDS next to one tile.
// Per tile a thread loads one 16-byte vector along the input's rows and writes it to the tile; after a barrier it gathers
// eight values down a tile column, looks them up and stores 16 bytes along the output's row; the next tile's vector is
// fetched before that second phase, so its latency passes behind the lookups.
template <class T, bool STREAM>
__global__ __launch_bounds__(LUT_BLOCK) void lut16_trv_kernel(const uint16_t* __restrict__ table, NdSpace<2> sp, EwPtrs<1> p, TrPlan<1> pl, uint32_t tiles) {
    using Cfg = TrvCfg<T>;
    constexpr int VEC = Cfg::VEC, TP = Cfg::TP, TL = Cfg::TL, PITCH = Cfg::PITCH;
    static_assert(TL * (TP / VEC) == LUT_BLOCK && TP * (TL / VEC) == LUT_BLOCK, "one vector per thread in either phase");
    extern __shared__ __attribute__((aligned(16))) uint16_t lut[];
    uint16_t* tile = lut + 65536;
    for (int i = threadIdx.x; i < (int)(LUT_BYTES / 16); i += LUT_BLOCK) ((lut_u4*)lut)[i] = ((const lut_u4*)table)[i];

    const int last = sp.ndims - 1, pd = pl.pdim, t = threadIdx.x;
    const uint32_t np = sp.dims[pd], nl = sp.dims[last];
    const int64_t sl = sp.strides[1][last], so = sp.strides[0][pd];
    const int jl1 = t / (TP / VEC), il1 = (t % (TP / VEC)) * VEC;      // phase 1: a vector of row jl1 of the tile
    const int il2 = t / (TL / VEC), jl2 = (t % (TL / VEC)) * VEC;      // phase 2: a vector of output row il2
    struct Tile { int64_t in, out; uint32_t i0, j0; };
    auto locate = [&](uint32_t b) {
        uint32_t tl, tp, outer;
        fd_divmod(b, pl.div_tiles_l, b, tl);
        fd_divmod(b, pl.div_tiles_p, outer, tp);
        if (pl.super) {            // the 8x8 groups of ew_trv_kernel
            constexpr uint32_t S = 8;
            const uint32_t lin = tp * pl.tiles_l + tl, per_row = pl.tiles_l / S, st = lin / (S * S), in = lin % (S * S);
            tp = (st / per_row) * S + in / S;
            tl = (st % per_row) * S + in % S;
        }
        Tile r;
        r.in = 0; r.out = 0;
        for (int d = last - 1; d >= 0; --d) {
            if (d == pd) continue;
            uint32_t q, c;
            fd_divmod(outer, sp.div[d], q, c);
            r.out += (int64_t)c * sp.strides[0][d];
            r.in += (int64_t)c * sp.strides[1][d];
            outer = q;
        }
        r.i0 = tp * TP; r.j0 = tl * TL;
        return r;
    };
    AVec<T, VEC> v;
    bool have = false;
    auto fetch = [&](const Tile& w) {
        const uint32_t i = w.i0 + il1, j = w.j0 + jl1;
        have = i < np && j < nl;
        if (have) v = ld_vec<STREAM>((const AVec<T, VEC>*)((const T*)p.in[0] + w.in + (int64_t)i + (int64_t)j * sl));
    };
    uint32_t b = blockIdx.x;
    Tile cur;
    if (b < tiles) { cur = locate(b); fetch(cur); }
    __syncthreads();               // the table is in place
    for (; b < tiles; b += gridDim.x) {
        if (have) {
            // 32-bit LDS writes: the row pitch is not a multiple of 16 bytes
            const uint32_t* w = (const uint32_t*)&v;
            uint32_t* dst = (uint32_t*)(tile + jl1 * PITCH + il1);
#pragma unroll
            for (int e = 0; e < 4; ++e) dst[e] = w[e];
        }
        __syncthreads();
        const Tile now = cur;
        if (b + gridDim.x < tiles) { cur = locate(b + gridDim.x); fetch(cur); }
        const uint32_t i = now.i0 + il2, j = now.j0 + jl2;
        if (i < np && j < nl) {
            AVec<T, VEC> o;
#pragma unroll
            for (int e = 0; e < VEC; ++e) o.v[e].bits = lut[tile[(jl2 + e) * PITCH + il2]];
            st_vec<STREAM>((AVec<T, VEC>*)((T*)p.out + now.out + (int64_t)i * so + (int64_t)j), o);
        }
        __syncthreads();           // the tile is free again
    }
}

template <class T>
struct TrvOverride<OpLut16<T>> {
    static bool launch(const NdSpace<2>& sp, const EwPtrs<1>& p, const TrPlan<1>& pl, size_t blocks, bool streams, const OpLut16<T>& op) {
        constexpr size_t LDS = LUT_BYTES + (size_t)TrvCfg<T>::TL * TrvCfg<T>::PITCH * sizeof(T);
        static bool attr_set[16][2] = {{false}};
        int dev = 0;
        if (pl.staged != 1u || blocks >= (1ull << 32) || hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return false;
        const int cus = lut16_cus(dev);
        if (!cus) return false;
        if (!attr_set[dev][streams]) {
            hipError_t e = streams ? hipFuncSetAttribute((const void*)lut16_trv_kernel<T, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS)
                                   : hipFuncSetAttribute((const void*)lut16_trv_kernel<T, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS);
            if (e != hipSuccess) { (void)hipGetLastError(); return false; }
            attr_set[dev][streams] = true;
        }
        const unsigned grid = (unsigned)std::min<size_t>((size_t)cus, blocks);
        if (streams) hipLaunchKernelGGL((lut16_trv_kernel<T, true>), dim3(grid), dim3(LUT_BLOCK), LDS, stream(), op.table, sp, p, pl, (uint32_t)blocks);
        else hipLaunchKernelGGL((lut16_trv_kernel<T, false>), dim3(grid), dim3(LUT_BLOCK), LDS, stream(), op.table, sp, p, pl, (uint32_t)blocks);
        MXH_LAUNCH_CHECK("lut16_trv");
        return true;
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
        static int cus[16] = {0};
        static bool attr_set[16][2] = {{false}};
        int dev = 0;
        (void)hipGetDevice(&dev);
        if (!cus[dev]) {
            hipDeviceProp_t prop;
            if (hipGetDeviceProperties(&prop, dev) != hipSuccess) return false;
            cus[dev] = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
        }
        const bool streams = ew_stream_bytes() != 0 && num_els * 4 >= ew_stream_bytes();
        if (!attr_set[dev][streams]) {
            hipError_t e = streams ? hipFuncSetAttribute((const void*)lut16_kernel<true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)LUT_BYTES)
                                   : hipFuncSetAttribute((const void*)lut16_kernel<false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)LUT_BYTES);
            if (e != hipSuccess) { (void)hipGetLastError(); return false; }
            attr_set[dev][streams] = true;
        }
        const size_t nvec = num_els / 8;
        const unsigned blocks = (unsigned)std::min<size_t>((size_t)cus[dev], cdiv(nvec, (size_t)LUT_BLOCK * 2));
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
