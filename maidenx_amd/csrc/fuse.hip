// The kernel behind a fused group of elementwise launches: every thread owns one vector (or element) of the shared
// index space and applies the group's members to it in order.
#include <cstring>

#include "elementwise.hpp"
#include "fuse.hpp"
#include "mxh.hpp"
#include "ops.hpp"

namespace mxh {

// the functor at position I of EwProgOps applied to a thread's elements (only those that map float to float are
// recorded; the others compile to nothing)
template <int I, int VEC>
__device__ __forceinline__ void fuse_case(const float (&a)[VEC], const float (&b)[VEC], float (&r)[VEC], const uint32_t (&payload)[2]) {
    if constexpr (I < EwProgOps::size) {
        using Op = typename TypeAt<I, EwProgOps>::type;
        if constexpr (std::is_same<typename Op::Out, float>::value && std::is_same<typename Op::In, float>::value && sizeof(Op) <= 8) {
            Op o;
            __builtin_memcpy((void*)&o, payload, sizeof(Op));
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                if constexpr (Op::NIN == 1) r[e] = o(a[e]);
                else r[e] = o(a[e], b[e]);
            }
        }
    }
}
#define MXH_FC(I) case I: fuse_case<I, VEC>(val[0], val[1], r.v, c.payload); break;
#define MXH_FC8(B) MXH_FC(B + 0) MXH_FC(B + 1) MXH_FC(B + 2) MXH_FC(B + 3) MXH_FC(B + 4) MXH_FC(B + 5) MXH_FC(B + 6) MXH_FC(B + 7)
static_assert(EwProgOps::size <= 64, "the dispatch below has 64 cases");

template <int VEC>
__global__ __launch_bounds__(EW_BLOCK) void ew_group_kernel(FuseGroup g) {
    // The group description is 1.6 KB of kernel arguments; read member by member it costs a scalar-cache miss per
    // member.  Copy it to LDS once (one memory latency) and walk it there.
    __shared__ FuseGroup sg;
    {
        typedef uint32_t Piece __attribute__((ext_vector_type(4)));
        typedef const __attribute__((address_space(4))) Piece* ArgPtr;
        ArgPtr src = (ArgPtr)__builtin_amdgcn_kernarg_segment_ptr();
        static_assert(sizeof(FuseGroup) % 16 == 0, "copied in 16-byte pieces");
        for (unsigned i = threadIdx.x; i < sizeof(FuseGroup) / 16; i += EW_BLOCK) ((Piece*)&sg)[i] = src[i];
    }
    __syncthreads();
    const size_t v = (size_t)blockIdx.x * EW_BLOCK + threadIdx.x;
    const bool tiny = g.tiny != 0;               // one block; every thread stays for the barriers
    if (!tiny && v >= g.nvec) return;
    // coordinates of this thread's first element over (outer, inner); one dim: everything is "inner"
    uint32_t c0 = 0, c1 = (uint32_t)v * VEC;
    uint32_t ndims = g.ndims;
    if (!tiny && ndims == 2) fd_divmod((uint32_t)v * VEC, g.div_inner, c0, c1);
    AVec<float, VEC> r;          // what the previous member wrote at this thread's elements
#pragma unroll
    for (int e = 0; e < VEC; ++e) r.v[e] = 0.0f;
    for (uint32_t k = 0; k < g.n; ++k) {
        const FuseCmd& c = sg.cmd[k];
        if (tiny) {
            if (k) __syncthreads();              // the member before may have written what this one reads, anywhere
            if (v >= c.nel) continue;
            ndims = c.ndims;
            c0 = 0;
            c1 = (uint32_t)v;
            if (ndims == 2) { c0 = (uint32_t)v / c.dims[1]; c1 = (uint32_t)v - c0 * c.dims[1]; }
        }
        const int inner = ndims == 2 ? 1 : 0;
        float val[2][VEC];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            if (j >= (int)c.nin) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) val[j][e] = 0.0f;
                continue;
            }
            if (c.fwd & (1u << j)) {         // the value is still in registers: no need to wait for the store and read it back
#pragma unroll
                for (int e = 0; e < VEC; ++e) val[j][e] = r.v[e];
                continue;
            }
            const int64_t s = c.is[j][inner];
            const float* src = (const float*)c.in[j] + (ndims == 2 ? (int64_t)c0 * c.is[j][0] : 0) + (int64_t)c1 * s;
            if (VEC > 1 && s == 1) {
                const AVec<float, VEC> t = *(const AVec<float, VEC>*)src;
#pragma unroll
                for (int e = 0; e < VEC; ++e) val[j][e] = t.v[e];
            } else if (s == 0) {
                const float t = src[0];
#pragma unroll
                for (int e = 0; e < VEC; ++e) val[j][e] = t;
            } else {
#pragma unroll
                for (int e = 0; e < VEC; ++e) val[j][e] = src[(int64_t)e * s];
            }
        }
        switch (__builtin_amdgcn_readfirstlane(c.op)) {      // uniform: one scalar dispatch per member, not per element
            MXH_FC8(0) MXH_FC8(8) MXH_FC8(16) MXH_FC8(24) MXH_FC8(32) MXH_FC8(40) MXH_FC8(48) MXH_FC8(56)
            default: break;
        }
        float* dst = (float*)c.out + (ndims == 2 ? (int64_t)c0 * c.os[0] : 0) + (int64_t)c1 * c.os[inner];
        if (VEC > 1) {
            *(AVec<float, VEC>*)dst = r;
        } else {
            dst[0] = r.v[0];
        }
    }
}

void fuse_launch(const FuseGroup& g, void* stream_) {
    const unsigned blocks = g.tiny ? 1u : cdiv(g.nvec, (size_t)EW_BLOCK);
    if (g.vec) hipLaunchKernelGGL(ew_group_kernel<4>, dim3(blocks), dim3(EW_BLOCK), 0, (hipStream_t)stream_, g);
    else hipLaunchKernelGGL(ew_group_kernel<1>, dim3(blocks), dim3(EW_BLOCK), 0, (hipStream_t)stream_, g);
    MXH_HIP(hipGetLastError());
}

}  // namespace mxh
