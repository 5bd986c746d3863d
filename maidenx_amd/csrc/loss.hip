// Fused mean-squared-error loss and SGD step.
//
// The reference's MSELoss (crates/maidenx_nn/src/losses/mse.rs:21-29) is four tensor ops - sub, pow(2), sum_all,
// div_scalar - and its backward six more (the scalar's division, a broadcast, mul_scalar(2), mul by the difference, and
// the `0 + g` of sub's sum_to_shape), each a launch and, on a [32,64,56,56] prediction, a pass over 25 MB.  Its SGD
// (crates/maidenx_nn/src/optimizers/sgd.rs:17-27) is mul_scalar and an in-place sub per parameter.  The kernels here
// apply the same element functions in the same order to values held in registers:
//   forward   loss = (sum over i of square(pred[i] - target[i])) / n              one read of pred and target
//   backward  grad_pred[i]   = 0 + (((g / n) * 2) * (pred[i] - target[i]))         one read of pred and target, one write
//             (g = grad_loss[0], or 1 when no grad_loss is given: the seed of backward(), never written anywhere)
//             grad_target[i] = 0 + (-(((g / n) * 2) * (pred[i] - target[i])))      (when asked for)
//   sgd       param[i] = param[i] - grad[i] * lr
// Every gradient and every updated parameter is bit for bit what the op-by-op sequence gives (f32, no fused
// multiply-add; the difference is recomputed instead of stored, which is the same value).  The loss itself is a sum
// of n terms: like every sum of this library it is added in a fixed tree of its own, within the f32 tolerance of a
// reduction of the op sequence's sum (which the reference adds in an order that changes from run to run).
// Contiguous f32 tensors of one shape; anything else stays with the separate ops.
// Inside a capture, at launch-bound sizes, the three join the fused chains (fuse.hpp): the step as an elementwise
// launch (OpSgdStep), the one-block loss as a stage of the serial phase, the backward pass as a member of the parallel one.
#include "elementwise.hpp"
#include "fuse.hpp"
#include "loss.hpp"
#include "mxh.hpp"
#include "ops.hpp"
#include "reduce_row.hpp"

namespace mxh {

constexpr int LB = MSE_THREADS;
static inline bool aligned16(const void* p) { return ((uintptr_t)p % 16) == 0; }
constexpr unsigned MSE_MAX_BLOCKS = 1024;

// blocks == 1: the loss itself; more: one partial per block
__global__ __launch_bounds__(LB) void mse_sum_kernel(const float* __restrict__ pred, const float* __restrict__ target, size_t n, unsigned blocks,
                                                     float* __restrict__ out, float count) {
    __shared__ float part[LB / WAVE];
    const float sum = mse_block_sum(pred, target, n, blockIdx.x, blocks, threadIdx.x, part);
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
    const float scale = mse_grad_scale(grad_loss ? grad_loss[0] : 1.0f, count);
    const AVec<float, VEC> p = ((const AVec<float, VEC>*)pred)[i], t = ((const AVec<float, VEC>*)target)[i];
    AVec<float, VEC> gp, gt;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
        gp.v[e] = mse_grad(scale, p.v[e], t.v[e]);
        if (WITH_TARGET) gt.v[e] = 0.0f + OpNeg<float>{}(OpMul<float>{}(scale, OpSub<float>{}(p.v[e], t.v[e])));
    }
    if (grad_pred) ((AVec<float, VEC>*)grad_pred)[i] = gp;
    if (WITH_TARGET) ((AVec<float, VEC>*)grad_target)[i] = gt;
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
        if (capture_open()) {       // a stage of the open chain's serial phase: the same device function, run by one work-group of 256
            const MseArgs a{pred, target, loss, (uint64_t)n};
            const Extent in[2] = {{(uintptr_t)pred, (uintptr_t)(pred + n)}, {(uintptr_t)target, (uintptr_t)(target + n)}};
            const Extent out{(uintptr_t)loss, (uintptr_t)(loss + 1)};
            if (fuse_record_tail(TAIL_MSE, 0, &a, sizeof(a), in, 2, out, 1)) return;
        }
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
    if (!pred || !target) { set_status(ERR_INVALID, "mse_loss_backward: null buffer"); return; }
    if (n == 0 || (!grad_pred && !grad_target)) return;
    if (!grad_loss && grad_pred && !grad_target) {
        // the seed of backward(): an elementwise launch of two inputs with the constant folded into the functor - inside a
        // capture it joins the fused chains, recorded and resident programs like any other
        const size_t dims = n, unit = 1;
        const size_t* ins[2] = {&unit, &unit};
        const void* inp[2] = {pred, target};
        ew_launch<OpMseGradUnit<float>>(n, 1, &dims, &unit, ins, grad_pred, inp, OpMseGradUnit<float>{(float)n});
        return;
    }
    const bool vec = n % 4 == 0 && aligned16(pred) && aligned16(target) && (!grad_pred || aligned16(grad_pred)) && (!grad_target || aligned16(grad_target));
    const size_t units = vec ? n / 4 : n;
    const dim3 grid((unsigned)cdiv(units, (size_t)LB));
    if (units >= (1ull << 31) * LB) { set_status(ERR_TOO_LARGE, "mse_loss_backward: too many elements"); return; }
    if (capture_open() && grad_pred && !grad_target && n > 256 && units < (size_t)EW_SMALL_BLOCKS * EW_BLOCK * EW_UNR) {
        // launch-bound sizes inside a capture: a member of the open chain's parallel phase (two inputs walked element for
        // element like any elementwise member, and the loss's gradient read by every thread)
        FuseCmd c;
        std::memset((void*)&c, 0, sizeof(c));
        c.out = grad_pred;
        c.in[0] = pred;
        c.in[1] = target;
        c.os[0] = c.is[0][0] = c.is[1][0] = 1;
        c.op = FUSE_OP_MSE_BACKWARD;
        c.nin = 2;
        c.nel = (uint32_t)n;
        std::memcpy(c.payload, (const void*)&grad_loss, sizeof(grad_loss));
        const Extent seed = grad_loss ? Extent{(uintptr_t)grad_loss, (uintptr_t)(grad_loss + 1)} : Extent{0, 0};
        if (fuse_record_mse_backward(c, vec, units, seed)) return;
    }
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
    // an elementwise launch of two inputs, written over the first: inside a capture it joins the fused chains like any other
    const size_t dims = n, unit = 1;
    const size_t* ins[2] = {&unit, &unit};
    const void* inp[2] = {param, grad};
    ew_launch<OpSgdStep<float>>(n, 1, &dims, &unit, ins, param, inp, OpSgdStep<float>{lr});
}
