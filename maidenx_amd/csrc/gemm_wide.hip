// matmul / matmul_backward for f64 and the integer dtypes (crates/maidenx_cuda/src/ops/matmul.rs:36-50 of the
// reference's declarations; semantics crates/maidenx_cpu/src/ops/matmul.rs:5-268).  There is no matrix instruction
// behind these: a 64 x 64 output tile per 256-thread block, operands staged through LDS in k-tiles of 16, a 4 x 4
// register tile per thread.  Every output element is accumulated by one thread with r ascending, multiply and add
// unfused, in the storage type - the reference's own order - so f64 results carry its bits and integer results wrap as
// its release build does.
#include "gemm_host.hpp"

namespace mxh {

template <class T> __device__ inline T wmac(T acc, T a, T b) {
    if constexpr (std::is_integral<T>::value) {
        using U = typename std::make_unsigned<T>::type;
        return (T)(U)((U)acc + (U)((U)a * (U)b));
    } else return acc + a * b;
}

constexpr int WT = 64, WK = 16;

template <class T>
__global__ __launch_bounds__(256) void gemm_wide_kernel(GemmArgs g) {
    __shared__ T xs[WK][WT + 1], ys[WK][WT + 1];
    const uint32_t t = threadIdx.x, tx = t % 16, ty = t / 16;
    const uint32_t b = blockIdx.z, i0 = blockIdx.y * WT, j0 = blockIdx.x * WT;
    const T* X = (const T*)g.X + (int64_t)b * g.xb;
    const T* Y = (const T*)g.Y + (int64_t)b * g.yb;
    // which index runs along consecutive threads when a tile is fetched: the one whose stride is 1
    const bool x_r_fast = g.xr == 1, y_r_fast = g.yr == 1 && g.yj != 1;
    T acc[4][4];
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int c = 0; c < 4; ++c) acc[a][c] = (T)0;
    for (uint32_t r0 = 0; r0 < g.R; r0 += WK) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const uint32_t e = t + 256 * q;                      // 1024 elements of each 64 x 16 operand tile
            uint32_t il, rl;
            if (x_r_fast) { rl = e % WK; il = e / WK; } else { il = e % WT; rl = e / WT; }
            const uint32_t i = i0 + il, r = r0 + rl;
            xs[rl][il] = (i < g.I && r < g.R) ? X[(int64_t)i * g.xi + (int64_t)r * g.xr] : (T)0;
            uint32_t jl, sl;
            if (y_r_fast) { sl = e % WK; jl = e / WK; } else { jl = e % WT; sl = e / WT; }
            const uint32_t j = j0 + jl, s = r0 + sl;
            ys[sl][jl] = (j < g.J && s < g.R) ? Y[(int64_t)s * g.yr + (int64_t)j * g.yj] : (T)0;
        }
        __syncthreads();
        const uint32_t kmax = g.R - r0 < (uint32_t)WK ? g.R - r0 : (uint32_t)WK;      // (zero padding would add `+ 0 * 0`: harmless for the
        for (uint32_t kk = 0; kk < kmax; ++kk) {                                      //  integers, but -0 + 0*0 is +0 in f64, so stop at R)
            T av[4], bv[4];
#pragma unroll
            for (int a = 0; a < 4; ++a) av[a] = xs[kk][ty + 16 * a];
#pragma unroll
            for (int c = 0; c < 4; ++c) bv[c] = ys[kk][tx + 16 * c];
#pragma unroll
            for (int a = 0; a < 4; ++a)
#pragma unroll
                for (int c = 0; c < 4; ++c) acc[a][c] = wmac(acc[a][c], av[a], bv[c]);
        }
        __syncthreads();
    }
    T* out = (T*)g.out + (size_t)b * g.I * g.J;
#pragma unroll
    for (int a = 0; a < 4; ++a) {
        const uint32_t i = i0 + ty + 16 * a;
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            const uint32_t j = j0 + tx + 16 * c;
            if (i < g.I && j < g.J) out[(size_t)i * g.J + j] = acc[a][c];
        }
    }
}

template <class T>
static void gemm_wide_dispatch(GemmArgs g) {
    if (g.batch == 0 || g.I == 0 || g.J == 0) return;
    if (g.batch > 65535) { set_status(ERR_TOO_LARGE, "matmul: more than 65535 batches for this dtype"); return; }
    const dim3 grid(cdiv(g.J, (uint32_t)WT), cdiv(g.I, (uint32_t)WT), g.batch);
    if (grid.y > 65535) { set_status(ERR_TOO_LARGE, "matmul: more than 65535 row tiles for this dtype"); return; }
    hipLaunchKernelGGL(gemm_wide_kernel<T>, grid, dim3(256), 0, stream(), g);
    MXH_LAUNCH_CHECK("gemm_wide");
}

}  // namespace mxh

using namespace mxh;

#define MXH_MATMUL_WIDE_FOR(T, SUF)                                                                         \
    extern "C" void hip_matmul_##SUF(size_t num_els, const size_t* md, const T* a, const T* b, T* c) { MXH_API; \
        matmul_fwd<T>(num_els, md, a, b, c, [](GemmArgs g) { gemm_wide_dispatch<T>(g); });                  \
    }                                                                                                       \
    extern "C" void hip_matmul_backward_##SUF(size_t na, size_t nb, const size_t* md, const T* go,          \
                                              const T* a, const T* b, T* ga, T* gb) { MXH_API;              \
        matmul_bwd<T>(na, nb, md, go, a, b, ga, gb, [](GemmArgs g) { gemm_wide_dispatch<T>(g); });          \
    }
MXH_MATMUL_WIDE_FOR(double, f64)
MXH_MATMUL_WIDE_FOR(uint8_t, u8)
MXH_MATMUL_WIDE_FOR(uint16_t, u16)
MXH_MATMUL_WIDE_FOR(uint32_t, u32)
MXH_MATMUL_WIDE_FOR(uint64_t, u64)
MXH_MATMUL_WIDE_FOR(int8_t, i8)
MXH_MATMUL_WIDE_FOR(int16_t, i16)
MXH_MATMUL_WIDE_FOR(int32_t, i32)
MXH_MATMUL_WIDE_FOR(int64_t, i64)
