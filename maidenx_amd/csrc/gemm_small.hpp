// Operand description of a matmul, the element codecs and the two kernels for very small products: shared by
// the GEMM dispatch and by the interpreter of recorded programs.
#pragma once
#include "mxh.hpp"

namespace mxh {

struct GemmArgs {
    const void* X;
    const void* Y;
    void* out;
    int64_t xb, xi, xr;   // element strides of X: batch, output row, reduction
    int64_t yb, yr, yj;   // element strides of Y: batch, reduction, output column
    uint32_t I, J, R, batch;
    uint32_t tiles_i, tiles_j;
    // split-K: the reduction is cut into `splits` chunks of r_chunk (a multiple of the k-tile); with splits > 1
    // every block writes its f32 partial tile to part[split][batch*I*J] and a second kernel folds them
    uint32_t splits, r_chunk;
    float* part;
};

template <class T> struct Elem;
template <> struct Elem<float> {
    static constexpr int VEC = 4;      // elements per 16-byte LDS fragment read
    static __device__ float ld(float v) { return v; }
    static __device__ float st(float v) { return v; }
    static __device__ float zero() { return 0.0f; }
};
template <> struct Elem<bf16_t> {
    static constexpr int VEC = 8;
    static __device__ float ld(bf16_t v) { return bf2f(v); }
    static __device__ bf16_t st(float v) { return f2bf(v); }
    static __device__ bf16_t zero() { return bf16_t{0}; }
};
template <> struct Elem<f16_t> {
    static constexpr int VEC = 8;
    static __device__ float ld(f16_t v) { return h2f(v); }
    static __device__ f16_t st(float v) { return f2h(v); }
    static __device__ f16_t zero() { return f16_t{0}; }
};

constexpr int GB = 256;          // threads per block of the small-shape kernels

// ---- small shapes -----------------------------------------------------------------------------------
// One thread per output element, r ascending, multiply and add unfused: the reference's own
// order, so f32 results are bit-identical to it.
template <class T>
__device__ __forceinline__ void gemm_thread_body(const GemmArgs& g, unsigned bid, unsigned tid) {
    size_t idx = (size_t)bid * GB + tid;
    size_t per = (size_t)g.I * g.J;
    if (idx >= per * g.batch) return;
    uint32_t b = (uint32_t)(idx / per);
    uint32_t rem = (uint32_t)(idx % per);
    uint32_t i = rem / g.J, j = rem % g.J;
    const T* x = (const T*)g.X + (int64_t)b * g.xb + (int64_t)i * g.xi;
    const T* y = (const T*)g.Y + (int64_t)b * g.yb + (int64_t)j * g.yj;
    float acc = 0.0f;
    for (uint32_t r = 0; r < g.R; ++r) acc = acc + Elem<T>::ld(x[(int64_t)r * g.xr]) * Elem<T>::ld(y[(int64_t)r * g.yr]);
    ((T*)g.out)[idx] = Elem<T>::st(acc);
}
template <class T>
__global__ __launch_bounds__(GB) void gemm_thread_kernel(GemmArgs g) { gemm_thread_body<T>(g, blockIdx.x, threadIdx.x); }

// One block per output element for a handful of outputs with a long reduction (the MLP's weight gradient:
// 3 outputs of 10000 terms): threads stride over r, waves fold by shuffles, the block by LDS, in a fixed order.
// `part`: 1024 / WAVE floats of LDS; every thread reaches the barrier.
template <class T>
__device__ __forceinline__ void gemm_blockdot_body(const GemmArgs& g, unsigned bid, unsigned tid, float* part) {
    const size_t idx = bid;
    const size_t per = (size_t)g.I * g.J;
    const uint32_t b = (uint32_t)(idx / per), rem = (uint32_t)(idx % per);
    const uint32_t i = rem / g.J, j = rem % g.J;
    const T* x = (const T*)g.X + (int64_t)b * g.xb + (int64_t)i * g.xi;
    const T* y = (const T*)g.Y + (int64_t)b * g.yb + (int64_t)j * g.yj;
    float acc = 0.0f;
    for (uint32_t r = tid; r < g.R; r += 1024) acc += Elem<T>::ld(x[(int64_t)r * g.xr]) * Elem<T>::ld(y[(int64_t)r * g.yr]);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, WAVE);
    if (tid % WAVE == 0) part[tid / WAVE] = acc;
    __syncthreads();
    if (tid == 0) {
        float sum = 0.0f;
#pragma unroll
        for (int w = 0; w < 1024 / WAVE; ++w) sum += part[w];
        ((T*)g.out)[idx] = Elem<T>::st(sum);
    }
}
template <class T>
__global__ __launch_bounds__(1024) void gemm_blockdot_kernel(GemmArgs g) {
    __shared__ float part[1024 / WAVE];
    gemm_blockdot_body<T>(g, blockIdx.x, threadIdx.x, part);
}

}  // namespace mxh
