// Device code of the fused MSE loss shared by its own kernels (loss.hip) and by the fused chains of a capture, whose
// serial phase runs the one-block sum as a stage and whose parallel phase has the backward pass as a member (fuse.hip).
#pragma once
#include <cstddef>
#include <cstdint>

#include "mxh.hpp"
#include "ops.hpp"
#include "reduce_row.hpp"

namespace mxh {

constexpr int MSE_THREADS = 256;

// argument block of the one-block sum as a stage of a chain's serial phase
struct MseArgs {
    const float* pred;
    const float* target;
    float* loss;
    uint64_t n;
};

// One block's share (block `block` of `blocks`) of the squared differences, folded to one value in thread 0; the 256
// threads of the block all call it.  `part`: MSE_THREADS / WAVE floats of LDS.  `active` false: a thread of a larger
// work-group that only takes part in the barrier (tid is then anything).
__device__ __forceinline__ float mse_block_sum(const float* pred, const float* target, size_t n, unsigned block, unsigned blocks, unsigned tid,
                                               float* part, bool active = true) {
    typedef float F4 __attribute__((ext_vector_type(4)));
    const size_t nvec = active ? n / 4 : 0;
    float a[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    const size_t stride = (size_t)blocks * MSE_THREADS;
    size_t v = (size_t)block * MSE_THREADS + tid;
    constexpr int U = 8;                                   // pairs of loads in flight (the terms are added in ascending v whatever U is)
    for (; v + (U - 1) * stride < nvec; v += U * stride) {
        F4 p[U], t[U];
#pragma unroll
        for (int k = 0; k < U; ++k) {
            p[k] = ((const F4*)pred)[v + k * stride];
            t[k] = ((const F4*)target)[v + k * stride];
        }
#pragma unroll
        for (int k = 0; k < U; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) a[e] = a[e] + OpSquare<float>{}(OpSub<float>{}(p[k][e], t[k][e]));
    }
    for (; v < nvec; v += stride) {
        const F4 p = ((const F4*)pred)[v], t = ((const F4*)target)[v];
#pragma unroll
        for (int e = 0; e < 4; ++e) a[e] = a[e] + OpSquare<float>{}(OpSub<float>{}(p[e], t[e]));
    }
    float acc = (a[0] + a[1]) + (a[2] + a[3]);
    if (active && block == 0 && tid < n % 4) {             // the last n % 4 elements
        const size_t i = nvec * 4 + tid;
        acc = acc + OpSquare<float>{}(OpSub<float>{}(pred[i], target[i]));
    }
    acc = wave_reduce<RSum>(acc);
    if (active && tid % WAVE == 0) part[tid / WAVE] = acc;
    __syncthreads();
    float sum = 0.0f;
    if (active && tid == 0) {
        sum = part[0];
#pragma unroll
        for (int w = 1; w < MSE_THREADS / WAVE; ++w) sum = sum + part[w];
    }
    return sum;
}

// the backward pass's element function: 0 + (((g / n) * 2) * (p - t)), each step rounded as the op sequence rounds it
__device__ __forceinline__ float mse_grad_scale(float grad_loss, float count) { return OpMulScalar<float>{2.0f}(OpDivScalar<float>{count}(grad_loss)); }
__device__ __forceinline__ float mse_grad(float scale, float p, float t) { return 0.0f + OpMul<float>{}(scale, OpSub<float>{}(p, t)); }

}  // namespace mxh
