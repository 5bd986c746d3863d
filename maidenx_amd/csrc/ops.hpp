// Element functions of the backend, written against the reference's CPU semantics
// (crates/maidenx_cpu/src/ops/{binary,unary}.rs).  f32 evaluates every step in f32 with no
// fused multiply-add (the translation unit is built with -ffp-contract=off); bf16 follows the
// `half` crate: arithmetic forms round after every operation, transcendental forms upcast,
// evaluate in f32 and round once.
#pragma once
#include <limits>
#include <type_traits>
#include "mathfn.hpp"
#include "mxh.hpp"

namespace mxh {

using bool_t = uint8_t;   // the reference's `bool` output buffers: one byte, 0 or 1

template <class T> struct Ar;
template <> struct Ar<float> {
    using T = float;
    static constexpr bool kFloat = true;
    static __device__ T zero() { return 0.0f; }
    static __device__ T inf() { return INFINITY; }
    static __device__ T from_f32(float v) { return v; }
    static __device__ float to_f32(T v) { return v; }
    static __device__ T add(T a, T b) { return a + b; }
    static __device__ T sub(T a, T b) { return a - b; }
    static __device__ T mul(T a, T b) { return a * b; }
    static __device__ T div(T a, T b) { return a / b; }
    static __device__ T neg(T a) { return -a; }
    static __device__ T max_(T a, T b) { return fmaxf(a, b); }   // f32::max — a NaN operand is ignored
    static __device__ T min_(T a, T b) { return fminf(a, b); }
};
template <> struct Ar<bf16_t> {
    using T = bf16_t;
    static constexpr bool kFloat = true;
    static __device__ T zero() { return T{0}; }
    static __device__ T inf() { return T{0x7F80}; }
    static __device__ T from_f32(float v) { return f2bf(v); }
    static __device__ float to_f32(T v) { return bf2f(v); }
    static __device__ T add(T a, T b) { return f2bf(bf2f(a) + bf2f(b)); }
    static __device__ T sub(T a, T b) { return f2bf(bf2f(a) - bf2f(b)); }
    static __device__ T mul(T a, T b) { return f2bf(bf2f(a) * bf2f(b)); }
    static __device__ T div(T a, T b) { return f2bf(bf2f(a) / bf2f(b)); }
    static __device__ T neg(T a) { return T{(uint16_t)(a.bits ^ 0x8000u)}; }
    static __device__ T max_(T a, T b) { return bf2f(a) > bf2f(b) ? a : b; }   // `if a > b { a } else { b }`
    static __device__ T min_(T a, T b) { return bf2f(a) < bf2f(b) ? a : b; }
};
template <> struct Ar<f16_t> {       // the `half` crate's f16: the same "f32 operation, round" scheme as bf16
    using T = f16_t;
    static constexpr bool kFloat = true;
    static __device__ T zero() { return T{0}; }
    static __device__ T inf() { return T{0x7C00}; }
    static __device__ T from_f32(float v) { return f2h(v); }
    static __device__ float to_f32(T v) { return h2f(v); }
    static __device__ T add(T a, T b) { return f2h(h2f(a) + h2f(b)); }
    static __device__ T sub(T a, T b) { return f2h(h2f(a) - h2f(b)); }
    static __device__ T mul(T a, T b) { return f2h(h2f(a) * h2f(b)); }
    static __device__ T div(T a, T b) { return f2h(h2f(a) / h2f(b)); }
    static __device__ T neg(T a) { return T{(uint16_t)(a.bits ^ 0x8000u)}; }
    static __device__ T max_(T a, T b) { return h2f(a) > h2f(b) ? a : b; }
    static __device__ T min_(T a, T b) { return h2f(a) < h2f(b) ? a : b; }
};
template <> struct Ar<double> {      // binary.rs:373,387,401,445-456,583,597
    using T = double;
    static constexpr bool kFloat = true;
    static __device__ T zero() { return 0.0; }
    static __device__ T inf() { return (double)INFINITY; }
    static __device__ T from_f32(float v) { return (double)v; }
    static __device__ float to_f32(T v) { return (float)v; }
    static __device__ T add(T a, T b) { return a + b; }
    static __device__ T sub(T a, T b) { return a - b; }
    static __device__ T mul(T a, T b) { return a * b; }
    static __device__ T div(T a, T b) { return a / b; }
    static __device__ T neg(T a) { return -a; }
    static __device__ T max_(T a, T b) { return fmax(a, b); }
    static __device__ T min_(T a, T b) { return fmin(a, b); }
};
// The reference's `bool` as an operand dtype: one byte holding 0 or 1 (binary.rs:374,388,402,457,584,598:
// add = or, sub = and, mul = xor, div = and, maximum = or, minimum = and).
struct b8_t { uint8_t bits; };
template <> struct Ar<b8_t> {
    using T = b8_t;
    static constexpr bool kFloat = false;
    static __device__ T add(T a, T b) { return T{(uint8_t)(a.bits | b.bits)}; }
    static __device__ T sub(T a, T b) { return T{(uint8_t)(a.bits & b.bits)}; }
    static __device__ T mul(T a, T b) { return T{(uint8_t)(a.bits ^ b.bits)}; }
    static __device__ T divq(T a, T b) { return T{(uint8_t)(a.bits & b.bits)}; }
    static __device__ T max_(T a, T b) { return T{(uint8_t)(a.bits | b.bits)}; }
    static __device__ T min_(T a, T b) { return T{(uint8_t)(a.bits & b.bits)}; }
};
// Integers saturate (binary.rs:375-382, 389-396, 403-410); a zero divisor gives 0 for 0/0 and otherwise the
// extreme value with the sign of the dividend, and MIN / -1 saturates to MAX (:458-578).
template <class I> struct IntAr {
    using T = I;
    static constexpr bool kFloat = false;
    static constexpr bool kSigned = std::is_signed<I>::value;
    static constexpr I kMax = std::numeric_limits<I>::max(), kMin = std::numeric_limits<I>::min();
    static __device__ T add(T a, T b) {
        T r;
        if (__builtin_add_overflow(a, b, &r)) return kSigned && b < 0 ? kMin : kMax;
        return r;
    }
    static __device__ T sub(T a, T b) {
        T r;
        if (__builtin_sub_overflow(a, b, &r)) return !kSigned || b > 0 ? kMin : kMax;
        return r;
    }
    static __device__ T mul(T a, T b) {
        T r;
        if (__builtin_mul_overflow(a, b, &r)) return kSigned && ((a < 0) != (b < 0)) ? kMin : kMax;
        return r;
    }
    static __device__ T divq(T a, T b) {
        if (b == 0) return a == 0 ? (T)0 : (kSigned && a < 0 ? kMin : kMax);
        if constexpr (kSigned) {
            if (a == kMin && b == (T)-1) return kMax;
        }
        return (T)(a / b);
    }
    static __device__ T max_(T a, T b) { return a > b ? a : b; }
    static __device__ T min_(T a, T b) { return a < b ? a : b; }
};
template <> struct Ar<uint8_t> : IntAr<uint8_t> {};
template <> struct Ar<uint16_t> : IntAr<uint16_t> {};
template <> struct Ar<uint32_t> : IntAr<uint32_t> {};
template <> struct Ar<uint64_t> : IntAr<uint64_t> {};
template <> struct Ar<int8_t> : IntAr<int8_t> {};
template <> struct Ar<int16_t> : IntAr<int16_t> {};
template <> struct Ar<int32_t> : IntAr<int32_t> {};
template <> struct Ar<int64_t> : IntAr<int64_t> {};

template <class T> __device__ inline float F(T v) { return Ar<T>::to_f32(v); }
// the value comparisons and zero tests are made on: f32 for the three float formats stored in 32 or 16 bits (as the
// reference's `half` types compare), the value itself for f64 and the integers, 0 / 1 for bool
template <class T> __device__ inline auto V(T v) {
    if constexpr (std::is_same<T, b8_t>::value) return (int)v.bits;
    else if constexpr (std::is_same<T, double>::value || std::is_integral<T>::value) return v;
    else return F(v);
}
template <class T> __device__ inline bool is_zero(T v) { return V(v) == 0; }

// ---- binary --------------------------------------------------------------------------------
#define MXH_BIN(NAME, OUT, EXPR)                                          \
    template <class T> struct NAME {                                      \
        using In = T; using Out = OUT; static constexpr int NIN = 2;      \
        __device__ Out operator()(T a, T b) const { using A = Ar<T>; (void)sizeof(A); return EXPR; } \
    };
MXH_BIN(OpAdd, T, A::add(a, b))
MXH_BIN(OpSub, T, A::sub(a, b))
MXH_BIN(OpMul, T, A::mul(a, b))
// b == 0 ⇒ (a == 0 ? 0 : +INF) — the sign of a is ignored and a NaN a gives +INF
template <class T> struct OpDiv {
    using In = T; using Out = T; static constexpr int NIN = 2;
    __device__ T operator()(T a, T b) const {
        using A = Ar<T>;
        if constexpr (A::kFloat) return is_zero(b) ? (is_zero(a) ? A::zero() : A::inf()) : A::div(a, b);
        else return A::divq(a, b);
    }
};
MXH_BIN(OpMaximum, T, A::max_(a, b))
MXH_BIN(OpMinimum, T, A::min_(a, b))
MXH_BIN(OpLogicalAnd, bool_t, (bool_t)(!is_zero(a) && !is_zero(b)))
MXH_BIN(OpLogicalOr, bool_t, (bool_t)(!is_zero(a) || !is_zero(b)))
MXH_BIN(OpLogicalXor, bool_t, (bool_t)(!is_zero(a) != !is_zero(b)))
MXH_BIN(OpEq, bool_t, (bool_t)(V(a) == V(b)))
MXH_BIN(OpNe, bool_t, (bool_t)(V(a) != V(b)))
MXH_BIN(OpLt, bool_t, (bool_t)(V(a) < V(b)))
MXH_BIN(OpLe, bool_t, (bool_t)(V(a) <= V(b)))
MXH_BIN(OpGt, bool_t, (bool_t)(V(a) > V(b)))
MXH_BIN(OpGe, bool_t, (bool_t)(V(a) >= V(b)))

// ---- unary ---------------------------------------------------------------------------------
// EXPR_F sees `x` as f32 and yields f32 (rounded once for bf16); EXPR_T, when given, works on
// the storage type with per-operation rounding.
#define MXH_UN_F(NAME, EXPR_F)                                            \
    template <class T> struct NAME {                                      \
        using In = T; using Out = T; static constexpr int NIN = 1;        \
        __device__ T operator()(T v) const { float x = F(v); return Ar<T>::from_f32(EXPR_F); } \
    };
#define MXH_UN_T(NAME, EXPR_T)                                            \
    template <class T> struct NAME {                                      \
        using In = T; using Out = T; static constexpr int NIN = 1;        \
        __device__ T operator()(T x) const { using A = Ar<T>; (void)sizeof(A); return EXPR_T; } \
    };

__device__ inline float gelu_f32(float x) {
    const float sqrt_2_over_pi = 0.7978845608028654f, coeff = 0.044715f;
    float tanh_arg = sqrt_2_over_pi * (x + coeff * x * x * x);
    return 0.5f * x * (1.0f + m_tanh(tanh_arg));
}

MXH_UN_T(OpNeg, A::neg(x))
MXH_UN_F(OpAbs, fabsf(x))
MXH_UN_F(OpSign, x > 0.0f ? 1.0f : (x < 0.0f ? -1.0f : 0.0f))
MXH_UN_T(OpSquare, A::mul(x, x))
MXH_UN_F(OpSqrt, sqrtf(x))
MXH_UN_T(OpRelu, F(x) > 0.0f ? x : A::zero())          // NaN → 0, −0 → +0
MXH_UN_F(OpSigmoid, 1.0f / (1.0f + m_exp(-x)))
MXH_UN_F(OpTanh, m_tanh(x))
MXH_UN_F(OpGelu, gelu_f32(x))
MXH_UN_F(OpSin, m_sin(x))
MXH_UN_F(OpCos, m_cos(x))
MXH_UN_F(OpTan, m_tan(x))
MXH_UN_F(OpLn, m_ln(x))
MXH_UN_F(OpLog10, m_log10(x))
MXH_UN_F(OpLog2, m_log2(x))
MXH_UN_F(OpExp, m_exp(x))
MXH_UN_F(OpExp10, m_pow(10.0f, x))
MXH_UN_F(OpExp2, m_exp2(x))
MXH_UN_F(OpSoftplus, m_ln(1.0f + m_exp(x)))
MXH_UN_F(OpRecip, 1.0f / x)
template <class T> struct OpLogicalNot {
    using In = T; using Out = bool_t; static constexpr int NIN = 1;
    __device__ bool_t operator()(T x) const { return (bool_t)is_zero(x); }
};

// SGD's update as one function of (parameter, gradient): p - g * lr, the product rounded before the difference is
// taken - mul_scalar, then sub (crates/maidenx_nn/src/optimizers/sgd.rs:17-27)
template <class T> struct OpSgdStep {
    using In = T; using Out = T; static constexpr int NIN = 2;
    T lr;
    __device__ T operator()(T p, T g) const { using A = Ar<T>; return A::sub(p, A::mul(g, lr)); }
};

// ---- unary with a constant of the input dtype --------------------------------------------------
#define MXH_UNC(NAME, OUT, EXPR)                                          \
    template <class T> struct NAME {                                      \
        using In = T; using Out = OUT; static constexpr int NIN = 1;      \
        T c;                                                              \
        __device__ Out operator()(T x) const { using A = Ar<T>; (void)sizeof(A); return EXPR; } \
    };
MXH_UNC(OpAddScalar, T, A::add(x, c))
MXH_UNC(OpSubScalar, T, A::sub(x, c))
MXH_UNC(OpMulScalar, T, A::mul(x, c))
MXH_UNC(OpDivScalar, T, is_zero(c) ? (is_zero(x) ? A::zero() : A::inf()) : A::div(x, c))
// The backward pass of the MSE loss when the gradient of the loss is the seed of backward(), 1: 0 + (((1 / n) * 2) * (p - t)),
// every step the functor of the op sequence (crates/maidenx_nn/src/losses/mse.rs:21-29 backwards: div_scalar, mul_scalar(2),
// mul, and the `0 + g` of sub's sum_to_shape)
template <class T> struct OpMseGradUnit {
    using In = T; using Out = T; static constexpr int NIN = 2;
    T count;
    __device__ T operator()(T p, T t) const {
        using A = Ar<T>;
        const T scale = OpMulScalar<T>{A::from_f32(2.0f)}(OpDivScalar<T>{count}(A::from_f32(1.0f)));
        return A::add(A::zero(), OpMul<T>{}(scale, OpSub<T>{}(p, t)));
    }
};
MXH_UNC(OpMaximumScalar, T, A::max_(x, c))
MXH_UNC(OpMinimumScalar, T, A::min_(x, c))
MXH_UNC(OpPow, T, A::from_f32(m_pow(F(x), F(c))))                      // (the entry point sends an exponent of 2 to OpSquare)
MXH_UNC(OpLeakyRelu, T, F(x) > 0.0f ? x : A::mul(c, x))
MXH_UNC(OpElu, T, F(x) > 0.0f ? x : A::from_f32(F(c) * (m_exp(F(x)) - 1.0f)))
MXH_UNC(OpEqScalar, bool_t, (bool_t)(F(x) == F(c)))
MXH_UNC(OpNeScalar, bool_t, (bool_t)(F(x) != F(c)))
MXH_UNC(OpLtScalar, bool_t, (bool_t)(F(x) < F(c)))
MXH_UNC(OpLeScalar, bool_t, (bool_t)(F(x) <= F(c)))
MXH_UNC(OpGtScalar, bool_t, (bool_t)(F(x) > F(c)))
MXH_UNC(OpGeScalar, bool_t, (bool_t)(F(x) >= F(c)))

// ---- functors without an arithmetic of their own ---------------------------------------------
template <class T> struct OpFill {     // output-only "unary": the input value is ignored
    using In = T; using Out = T; static constexpr int NIN = 1;
    T c;
    __device__ T operator()(T) const { return c; }
};
template <class T> struct OpIdentity {
    using In = T; using Out = T; static constexpr int NIN = 1;
    __device__ T operator()(T x) const { return x; }
};
// lhs = rhs through the in-place path (index_put_): the old value is not used
template <class T> struct OpAssign {
    using In = T; using Out = T; static constexpr int NIN = 2;
    __device__ T operator()(T, T b) const { return b; }
};
// `0 + x`: what a sum_to_shape that keeps every dim does through its zero-initialised cells (-0 -> +0).
// The 16-bit forms live with the reductions, whose rounding helpers they use.
template <class T> struct OpZeroPlus;
template <> struct OpZeroPlus<float> {
    using In = float; using Out = float; static constexpr int NIN = 1;
    __device__ float operator()(float x) const { return 0.0f + x; }
};

}  // namespace mxh
