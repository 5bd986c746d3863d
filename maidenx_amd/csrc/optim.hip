// Fused Adam step.  The reference's optimizer (crates/maidenx_nn/src/optimizers/adam.rs:34-88) updates every
// parameter with fourteen tensor ops, each a pass over memory:
//     m = m*b1 + g*(1-b1);  v = v*b2 + (g*g)*(1-b2);  m_hat = m / c1;  v_hat = v / c2;
//     p -= (m_hat / (sqrt(v_hat) + eps)) * lr_t
// This kernel applies the same element functions in the same order to values held in registers - one read of
// p, g, m, v and one write of p, m, v instead of some forty passes - so every intermediate is rounded exactly as
// the op-by-op sequence rounds it (f32: no fused multiply-add; bf16 / f16: one rounding per op) and the results are
// bit-identical to it.  The eight scalars are what the reference hands to its *_scalar ops, already in the tensor's
// dtype: computing them (its bias terms use beta^(t+1), in the precision of its Scalar arithmetic) stays with the
// caller.  Contiguous tensors only; a caller with a strided parameter uses the separate ops.
#include "elementwise.hpp"
#include "mxh.hpp"
#include "ops.hpp"

namespace mxh {

template <class T>
struct AdamScalars {
    T beta1, one_minus_beta1, beta2, one_minus_beta2, bias1, bias2, epsilon, lr_t;
};

template <class T>
__device__ __forceinline__ void adam_element(T& p, T g, T& m, T& v, const AdamScalars<T>& s) {
    m = OpAdd<T>{}(OpMulScalar<T>{s.beta1}(m), OpMulScalar<T>{s.one_minus_beta1}(g));
    v = OpAdd<T>{}(OpMulScalar<T>{s.beta2}(v), OpMulScalar<T>{s.one_minus_beta2}(OpSquare<T>{}(g)));
    const T m_hat = OpDivScalar<T>{s.bias1}(m);
    const T v_hat = OpDivScalar<T>{s.bias2}(v);
    const T step = OpDiv<T>{}(m_hat, OpAddScalar<T>{s.epsilon}(OpSqrt<T>{}(v_hat)));
    p = OpSub<T>{}(p, OpMulScalar<T>{s.lr_t}(step));
}

constexpr int AB = 256;

template <class T, int VEC>
__global__ __launch_bounds__(AB) void adam_step_kernel(size_t nvec, T* __restrict__ param, const T* __restrict__ grad, T* __restrict__ m,
                                                       T* __restrict__ v, AdamScalars<T> s) {
    const size_t i = (size_t)blockIdx.x * AB + threadIdx.x;
    if (i >= nvec) return;
    AVec<T, VEC> p = ((const AVec<T, VEC>*)param)[i], g = ((const AVec<T, VEC>*)grad)[i];
    AVec<T, VEC> mm = ((const AVec<T, VEC>*)m)[i], vv = ((const AVec<T, VEC>*)v)[i];
#pragma unroll
    for (int e = 0; e < VEC; ++e) adam_element<T>(p.v[e], g.v[e], mm.v[e], vv.v[e], s);
    ((AVec<T, VEC>*)param)[i] = p;
    ((AVec<T, VEC>*)m)[i] = mm;
    ((AVec<T, VEC>*)v)[i] = vv;
}

template <class T>
void adam_step(size_t n, T* param, const T* grad, T* m, T* v, const AdamScalars<T>& s) {
    if (n == 0) return;
    if (!param || !grad || !m || !v) { set_status(ERR_INVALID, "adam_step: null buffer"); return; }
    constexpr int VEC = 16 / sizeof(T);
    auto al = [](const void* p) { return ((uintptr_t)p & 15u) == 0; };
    if (n % VEC == 0 && al(param) && al(grad) && al(m) && al(v)) {
        const size_t nvec = n / VEC;
        hipLaunchKernelGGL((adam_step_kernel<T, VEC>), dim3((unsigned)cdiv(nvec, AB)), dim3(AB), 0, stream(), nvec, param, grad, m, v, s);
    } else {
        hipLaunchKernelGGL((adam_step_kernel<T, 1>), dim3((unsigned)cdiv(n, AB)), dim3(AB), 0, stream(), n, param, grad, m, v, s);
    }
    MXH_LAUNCH_CHECK("adam_step");
}

}  // namespace mxh

using namespace mxh;

#define MXH_ADAM_FOR(T, SUF)                                                                                               \
    extern "C" void hip_adam_step_##SUF(size_t n, T* param, const T* grad, T* m, T* v, T beta1, T one_minus_beta1, T beta2,  \
                                        T one_minus_beta2, T bias1, T bias2, T epsilon, T lr_t) { MXH_API;                 \
        adam_step<T>(n, param, grad, m, v, AdamScalars<T>{beta1, one_minus_beta1, beta2, one_minus_beta2, bias1, bias2, epsilon, lr_t}); \
    }
MXH_ADAM_FOR(float, f32)
MXH_ADAM_FOR(bf16_t, bf16)
MXH_ADAM_FOR(f16_t, f16)
