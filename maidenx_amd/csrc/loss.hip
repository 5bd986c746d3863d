// Fused mean-squared-error loss and SGD step.
//
// The reference's MSELoss (crates/maidenx_nn/src/losses/mse.rs:21-29) is four tensor ops - sub, pow(2), sum_all,
// div_scalar - and its backward six more (the scalar's division, a broadcast, mul_scalar(2), mul by the difference, and
// the `0 + g` of sub's sum_to_shape), each a launch and, on a [32,64,56,56] prediction, a pass over 25 MB.  Its SGD
// (crates/maidenx_nn/src/optimizers/sgd.rs:17-27) is mul_scalar and an in-place sub per parameter.  The kernels here
// apply the same element functions in the same order to values held in registers:
//   forward   loss = (sum over i of square(pred[i] - target[i])) / n              one read of pred and target
//   backward  grad_pred[i]   = 0 + (((g / n) * 2) * (pred[i] - target[i]))         one read of pred and target, one write
//             grad_target[i] = 0 + (-(((g / n) * 2) * (pred[i] - target[i])))      (when asked for)
//   sgd       param[i] = param[i] - grad[i] * lr
// Every gradient and every updated parameter is bit for bit what the op-by-op sequence gives (f32, no fused
// multiply-add; the difference is recomputed instead of stored, which is the same value).  The loss itself is a sum
// of n terms: like every sum of this library it is added in a fixed tree of its own, within the f32 tolerance of a
// reduction of the op sequence's sum (which the reference adds in an order that changes from run to run).
// Contiguous f32 tensors of one shape; anything else stays with the separate ops.
#include "elementwise.hpp"
#include "mxh.hpp"
#include "ops.hpp"
#include "reduce_row.hpp"

namespace mxh {

constexpr int LB = 256;
static inline bool aligned16(const void* p) { return ((uintptr_t)p % 16) == 0; }
constexpr unsigned MSE_MAX_BLOCKS = 1024;

// one block's share of the squared differences, folded to one value in thread 0
__device__ __forceinline__ float mse_block_sum(const float* __restrict__ pred, const float* __restrict__ target, size_t n, unsigned blocks, float* part) {
    typedef float F4 __attribute__((ext_vector_type(4)));
    const size_t nvec = n / 4;
    float a[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    const size_t stride = (size_t)blocks * LB;
    size_t v = (size_t)blockIdx.x * LB + threadIdx.x;
    for (; v + 3 * stride < nvec; v += 4 * stride) {      // four pairs of loads in flight
        F4 p[4], t[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            p[k] = ((const F4*)pred)[v + k * stride];
            t[k] = ((const F4*)target)[v + k * stride];
        }
#pragma unroll
        for (int k = 0; k < 4; ++k)
#pragma unroll
            for (int e = 0; e < 4; ++e) a[e] = a[e] + OpSquare<float>{}(OpSub<float>{}(p[k][e], t[k][e]));
    }
    for (; v < nvec; v += stride) {
        const F4 p = ((const F4*)pred)[v], t = ((const F4*)target)[v];
#pragma unroll
        for (int e = 0; e < 4; ++e) a[e] = a[e] + OpSquare<float>{}(OpSub<float>{}(p[e], t[e]));
    }
    float acc = (a[0] + a[1]) + (a[2] + a[3]);
    if (blockIdx.x == 0 && threadIdx.x < n % 4) {          // the last n % 4 elements
        const size_t i = nvec * 4 + threadIdx.x;
        acc = acc + OpSquare<float>{}(OpSub<float>{}(pred[i], target[i]));
    }
    acc = wave_reduce<RSum>(acc);
    if (threadIdx.x % WAVE == 0) part[threadIdx.x / WAVE] = acc;
    __syncthreads();
    float sum = 0.0f;
    if (threadIdx.x == 0) {
        sum = part[0];
#pragma unroll
        for (int w = 1; w < LB / WAVE; ++w) sum = sum + part[w];
    }
    return sum;
}
// blocks == 1: the loss itself; more: one partial per block
__global__ __launch_bounds__(LB) void mse_sum_kernel(const float* __restrict__ pred, const float* __restrict__ target, size_t n, unsigned blocks,
                                                     float* __restrict__ out, float count) {
    __shared__ float part[LB / WAVE];
    const float sum = mse_block_sum(pred, target, n, blocks, part);
    if (threadIdx.x == 0) out[blockIdx.x] = blocks == 1 ? OpDivScalar<float>{count}(sum) : sum;
}
// the blocks' partials in block order, then the division
__global__ __launch_bounds__(LB) void mse_fold_kernel(const float* __restrict__ partials, unsigned blocks, float* __restrict__ loss, float count) {
    __shared__ float part[LB / WAVE];
    float acc = 0.0f;
    for (unsigned i = threadIdx.x; i < blocks; i += LB) acc = acc + partials[i];
    acc = wave_reduce<RSum>(acc);
    if (threadIdx.x % WAVE == 0) part[threadIdx.x / WAVE] = acc;
    __syncthreads();
    if (threadIdx.x == 0) {
        float sum = part[0];
#pragma unroll
        for (int w = 1; w < LB / WAVE; ++w) sum = sum + part[w];
        loss[0] = OpDivScalar<float>{count}(sum);
    }
}

template <int VEC, bool WITH_TARGET>
__global__ __launch_bounds__(LB) void mse_backward_kernel(size_t nunits, const float* __restrict__ pred, const float* __restrict__ target,
                                                          const float* __restrict__ grad_loss, float* __restrict__ grad_pred,
                                                          float* __restrict__ grad_target, float count) {
    const size_t i = (size_t)blockIdx.x * LB + threadIdx.x;
    if (i >= nunits) return;
    // the scalar chain of the op sequence: div_scalar's backward, then pow's mul_scalar(2)
    const float scale = OpMulScalar<float>{2.0f}(OpDivScalar<float>{count}(grad_loss[0]));
    const AVec<float, VEC> p = ((const AVec<float, VEC>*)pred)[i], t = ((const AVec<float, VEC>*)target)[i];
    AVec<float, VEC> gp, gt;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
        const float u = OpMul<float>{}(scale, OpSub<float>{}(p.v[e], t.v[e]));
        gp.v[e] = 0.0f + u;
        if (WITH_TARGET) gt.v[e] = 0.0f + OpNeg<float>{}(u);
    }
    if (grad_pred) ((AVec<float, VEC>*)grad_pred)[i] = gp;
    if (WITH_TARGET) ((AVec<float, VEC>*)grad_target)[i] = gt;
}

template <int VEC>
__global__ __launch_bounds__(LB) void sgd_step_kernel(size_t nunits, float* __restrict__ param, const float* __restrict__ grad, float lr) {
    const size_t i = (size_t)blockIdx.x * LB + threadIdx.x;
    if (i >= nunits) return;
    AVec<float, VEC> p = ((const AVec<float, VEC>*)param)[i];
    const AVec<float, VEC> g = ((const AVec<float, VEC>*)grad)[i];
#pragma unroll
    for (int e = 0; e < VEC; ++e) p.v[e] = OpSub<float>{}(p.v[e], OpMulScalar<float>{lr}(g.v[e]));
    ((AVec<float, VEC>*)param)[i] = p;
}

}  // namespace mxh

using namespace mxh;

extern "C" void hip_mse_loss_f32(size_t n, const float* pred, const float* target, float* loss) { MXH_API;
    if (!pred || !target || !loss) { set_status(ERR_INVALID, "mse_loss: null buffer"); return; }
    if (n == 0) { set_status(ERR_INVALID, "mse_loss: no elements"); return; }
    if (!aligned16(pred) || !aligned16(target)) { set_status(ERR_INVALID, "mse_loss: operands must be 16-byte aligned"); return; }
    // one block up to 64 K elements (a launch-bound size: the second launch would cost more than it saves), else enough
    // blocks for the chip, each with at least 4096 elements
    unsigned blocks = 1;
    if (n > 65536) blocks = (unsigned)std::min<size_t>(MSE_MAX_BLOCKS, cdiv(n, (size_t)4096));
    if (blocks == 1) {
        hipLaunchKernelGGL(mse_sum_kernel, dim3(1), dim3(LB), 0, stream(), pred, target, n, 1u, loss, (float)n);
        MXH_LAUNCH_CHECK("mse_sum");
        return;
    }
    float* part = (float*)scratch(MSE_MAX_BLOCKS * sizeof(float));
    if (!part) return;
    hipLaunchKernelGGL(mse_sum_kernel, dim3(blocks), dim3(LB), 0, stream(), pred, target, n, blocks, part, (float)n);
    MXH_LAUNCH_CHECK("mse_sum");
    hipLaunchKernelGGL(mse_fold_kernel, dim3(1), dim3(LB), 0, stream(), part, blocks, loss, (float)n);
    MXH_LAUNCH_CHECK("mse_fold");
}

extern "C" void hip_mse_loss_backward_f32(size_t n, const float* pred, const float* target, const float* grad_loss, float* grad_pred,
                                          float* grad_target) { MXH_API;
    if (!pred || !target || !grad_loss) { set_status(ERR_INVALID, "mse_loss_backward: null buffer"); return; }
    if (n == 0 || (!grad_pred && !grad_target)) return;
    const bool vec = n % 4 == 0 && aligned16(pred) && aligned16(target) && (!grad_pred || aligned16(grad_pred)) && (!grad_target || aligned16(grad_target));
    const size_t units = vec ? n / 4 : n;
    const dim3 grid((unsigned)cdiv(units, (size_t)LB));
    if (units >= (1ull << 31) * LB) { set_status(ERR_TOO_LARGE, "mse_loss_backward: too many elements"); return; }
    if (vec) {
        if (grad_target) hipLaunchKernelGGL((mse_backward_kernel<4, true>), grid, dim3(LB), 0, stream(), units, pred, target, grad_loss, grad_pred, grad_target, (float)n);
        else hipLaunchKernelGGL((mse_backward_kernel<4, false>), grid, dim3(LB), 0, stream(), units, pred, target, grad_loss, grad_pred, grad_target, (float)n);
    } else {
        if (grad_target) hipLaunchKernelGGL((mse_backward_kernel<1, true>), grid, dim3(LB), 0, stream(), units, pred, target, grad_loss, grad_pred, grad_target, (float)n);
        else hipLaunchKernelGGL((mse_backward_kernel<1, false>), grid, dim3(LB), 0, stream(), units, pred, target, grad_loss, grad_pred, grad_target, (float)n);
    }
    MXH_LAUNCH_CHECK("mse_backward");
}

extern "C" void hip_sgd_step_f32(size_t n, float* param, const float* grad, float lr) { MXH_API;
    if (!param || !grad) { set_status(ERR_INVALID, "sgd_step: null buffer"); return; }
    if (n == 0) return;
    const bool vec = n % 4 == 0 && aligned16(param) && aligned16(grad);
    const size_t units = vec ? n / 4 : n;
    if (units >= (1ull << 31) * LB) { set_status(ERR_TOO_LARGE, "sgd_step: too many elements"); return; }
    const dim3 grid((unsigned)cdiv(units, (size_t)LB));
    if (vec) hipLaunchKernelGGL(sgd_step_kernel<4>, grid, dim3(LB), 0, stream(), units, param, grad, lr);
    else hipLaunchKernelGGL(sgd_step_kernel<1>, grid, dim3(LB), 0, stream(), units, param, grad, lr);
    MXH_LAUNCH_CHECK("sgd_step");
}
