// Unary element functions for f64, bool and the integers, after crates/maidenx_cpu/src/ops/unary.rs (line numbers at
// each group).  f64 has every form of the family (the transcendental ones through the device math library); bool and
// the integers have the forms the reference gives them; the integer `pow` (a float `powf` and a cast in the reference)
// is evaluated in exact integer arithmetic and rounded the way a correctly rounded `powf` and the cast would.
// Integer negation, absolute value and square wrap on overflow, as the reference's release build does (its debug
// build panics there); the scalar add / sub / mul saturate like the binary forms.
#pragma once
#include "cast.hpp"
#include "ops.hpp"

namespace mxh {

template <class T> struct Wide;

template <> struct Wide<double> {
    using T = double;
    static __device__ T neg(T x) { return -x; }                                       // unary.rs:125
    static __device__ T abs(T x) { return fabs(x); }                                  // :135
    static __device__ T sign(T x) { return x > 0.0 ? 1.0 : (x < 0.0 ? -1.0 : 0.0); }  // :151-157
    static __device__ T square(T x) { return x * x; }                                 // :207
    static __device__ T sqrt(T x) { return ::sqrt(x); }                               // :221
    static __device__ T relu(T x) { return x > 0.0 ? x : 0.0; }                       // :235
    static __device__ T recip(T x) { return 1.0 / x; }                                // :355
    static __device__ bool_t logical_not(T x) { return (bool_t)(x == 0.0); }          // :360
    static __device__ T add_scalar(T x, T c) { return x + c; }                        // :375
    static __device__ T sub_scalar(T x, T c) { return x - c; }
    static __device__ T mul_scalar(T x, T c) { return x * c; }
    static __device__ T div_scalar(T x, T c) { return c == 0.0 ? (x == 0.0 ? 0.0 : (double)INFINITY) : x / c; }      // :443-451
    static __device__ T maximum_scalar(T x, T c) { return fmax(x, c); }               // :537
    static __device__ T minimum_scalar(T x, T c) { return fmin(x, c); }
    static __device__ T leaky_relu(T x, T a) { return x > 0.0 ? x : a * x; }          // :585-589
    // transcendental forms (unary.rs:253, 263, 274-279, 295-355, 563, 611-617): the device math library's double
    // routines, each step a separate f64 operation as in the reference; results within 2 ulp of the host libm's
    static __device__ T sigmoid(T x) { return 1.0 / (1.0 + ::exp(-x)); }
    static __device__ T tanh(T x) { return ::tanh(x); }
    static __device__ T gelu(T x) {
        const T sqrt_2_over_pi = 0.7978845608028654, coeff = 0.044715;
        const T tanh_arg = sqrt_2_over_pi * (x + coeff * x * x * x);
        return 0.5 * x * (1.0 + ::tanh(tanh_arg));
    }
    static __device__ T sin(T x) { return ::sin(x); }
    static __device__ T cos(T x) { return ::cos(x); }
    static __device__ T tan(T x) { return ::tan(x); }
    static __device__ T ln(T x) { return ::log(x); }
    static __device__ T log10(T x) { return ::log10(x); }
    static __device__ T log2(T x) { return ::log2(x); }
    static __device__ T exp(T x) { return ::exp(x); }
    static __device__ T exp10(T x) { return ::pow(10.0, x); }
    static __device__ T exp2(T x) { return ::exp2(x); }
    static __device__ T softplus(T x) { return ::log(1.0 + ::exp(x)); }
    static __device__ T pow(T x, T c) { return ::pow(x, c); }
    static __device__ T elu(T x, T a) { return x > 0.0 ? x : a * (::exp(x) - 1.0); }
};

template <class I> struct WideInt {                       // unary.rs:127-130, 137-140, 159-198, 209-216, 223-230, 362-369
    using T = I;
    using U = typename std::make_unsigned<I>::type;
    static __device__ T neg(T x) { return (T)(U)((U)0 - (U)x); }
    static __device__ T abs(T x) { return x < 0 ? neg(x) : x; }
    static __device__ T sign(T x) { return x > 0 ? (T)1 : (x < 0 ? (T)-1 : (T)0); }
    static __device__ T square(T x) {
        if constexpr (sizeof(T) == 8) return (T)((U)x * (U)x);
        else return (T)(U)((uint32_t)(U)x * (uint32_t)(U)x);
    }
    // `(x as f32).sqrt() as T` (i64: f64), of the absolute value for the signed types
    static __device__ T sqrt(T x) {
        const T a = std::is_signed<T>::value ? abs(x) : x;
        if constexpr (std::is_same<T, int64_t>::value) return float_to_int<T>(::sqrt((double)a));
        else return float_to_int<T>(sqrtf((float)a));
    }
    // `(x as f64).powf(c as f64) as T` (u8 through f32), unary.rs:565-572.  Base and exponent are integers, so the power
    // is an integer, or for c < 0 a fraction that the cast truncates; no floating-point pow is evaluated.  The exact
    // power is formed in 128 bits and abandoned once it passes 2^64 (the cast saturates there anyway), rounded to f64 as
    // a correctly rounded pow returns it (exact below 2^53, which covers every non-saturating result of the types
    // narrower than 64 bits), and cast with Rust's `as` (toward zero, saturating).  A 64-bit base or exponent is first
    // rounded to f64 like the reference's `as f64`.
    static __device__ T pow(T x, T c) {
        using L = std::numeric_limits<T>;
        const bool xneg = x < 0, cneg = c < 0;
        uint64_t ax = xneg ? (uint64_t)(U)((U)0 - (U)x) : (uint64_t)(U)x;        // (back to U before widening: the subtraction is done in int)
        uint64_t ac = cneg ? (uint64_t)(U)((U)0 - (U)c) : (uint64_t)(U)c;
        unsigned __int128 base = ax;
        bool odd = (ac & 1) != 0;
        if constexpr (sizeof(T) == 8) {
            // the operands as f64: above 2^53 they are rounded to even multiples of a power of two
            const double bd = (double)ax;
            base = bd >= 18446744073709551616.0 ? ((unsigned __int128)1 << 64) : (unsigned __int128)(uint64_t)bd;
            if (ac > (1ull << 53)) { odd = false; }
        }
        if (ac == 0) return (T)1;                                    // pow(x, 0) = 1 for every x
        const bool neg = xneg && odd;
        if (cneg) {                                                  // 1 / |x|^|c|
            if (base == 0) return L::max();                          // pow(0, negative) = +inf
            if (base == 1) return neg ? (T)-1 : (T)1;
            return (T)0;
        }
        if (base == 0) return (T)0;
        if (base == 1) return neg ? (T)-1 : (T)1;
        unsigned __int128 p = 1, b = base;
        bool over = ac >= 64 || (base >> 64) != 0;                   // base >= 2: the 64th power is already 2^64 or more
        for (uint64_t e = ac; e != 0 && !over; e >>= 1) {
            if ((b >> 64) != 0) { over = true; break; }              // b enters the product at the top bit of e at the latest
            if (e & 1) { p *= b; if ((p >> 64) != 0) over = true; }
            b *= b;
        }
        double d = over ? 1.0e300 : (double)(uint64_t)p;             // (the integer to f64 conversion rounds to nearest even)
        if (neg) d = -d;
        return float_to_int<T>(d);
    }
    static __device__ bool_t logical_not(T x) { return (bool_t)(x == 0); }
    static __device__ T add_scalar(T x, T c) { return Ar<T>::add(x, c); }             // :377-384: saturating, like the binary forms
    static __device__ T sub_scalar(T x, T c) { return Ar<T>::sub(x, c); }
    static __device__ T mul_scalar(T x, T c) { return Ar<T>::mul(x, c); }
    static __device__ T div_scalar(T x, T c) { return Ar<T>::divq(x, c); }            // :453-533
    static __device__ T maximum_scalar(T x, T c) { return x > c ? x : c; }
    static __device__ T minimum_scalar(T x, T c) { return x < c ? x : c; }
};
template <> struct Wide<uint8_t> : WideInt<uint8_t> {};
template <> struct Wide<uint16_t> : WideInt<uint16_t> {};
template <> struct Wide<uint32_t> : WideInt<uint32_t> {};
template <> struct Wide<uint64_t> : WideInt<uint64_t> {};
template <> struct Wide<int8_t> : WideInt<int8_t> {};
template <> struct Wide<int16_t> : WideInt<int16_t> {};
template <> struct Wide<int32_t> : WideInt<int32_t> {};
template <> struct Wide<int64_t> : WideInt<int64_t> {};

// bool (unary.rs:126 neg = not; :136, 158, 208, 222, 236, 254, 264 identity; :361; scalar forms :376 or, :390 xor,
// :404 and, :452 and, :538 or, :552 and, :564 pow = x)
template <> struct Wide<b8_t> {
    using T = b8_t;
    static __device__ T neg(T x) { return T{(uint8_t)(x.bits ^ 1u)}; }
    static __device__ T same(T x) { return x; }
    static __device__ bool_t logical_not(T x) { return (bool_t)(x.bits == 0); }
    static __device__ T add_scalar(T x, T c) { return T{(uint8_t)(x.bits | c.bits)}; }
    static __device__ T sub_scalar(T x, T c) { return T{(uint8_t)(x.bits ^ c.bits)}; }
    static __device__ T mul_scalar(T x, T c) { return T{(uint8_t)(x.bits & c.bits)}; }
    static __device__ T div_scalar(T x, T c) { return T{(uint8_t)(x.bits & c.bits)}; }
    static __device__ T maximum_scalar(T x, T c) { return T{(uint8_t)(x.bits | c.bits)}; }
    static __device__ T minimum_scalar(T x, T c) { return T{(uint8_t)(x.bits & c.bits)}; }
    static __device__ T pow(T x, T) { return x; }
};

#define MXH_W1(NAME, FN)                                                                       \
    template <class T> struct W##NAME {                                                        \
        using In = T; using Out = decltype(Wide<T>::FN(T{})); static constexpr int NIN = 1;    \
        __device__ Out operator()(T x) const { return Wide<T>::FN(x); }                        \
    };
#define MXH_W1C(NAME, FN)                                                                      \
    template <class T> struct W##NAME {                                                        \
        using In = T; using Out = decltype(Wide<T>::FN(T{}, T{})); static constexpr int NIN = 1; \
        T c;                                                                                   \
        __device__ Out operator()(T x) const { return Wide<T>::FN(x, c); }                     \
    };
MXH_W1(Neg, neg) MXH_W1(Abs, abs) MXH_W1(Sign, sign) MXH_W1(Square, square) MXH_W1(Sqrt, sqrt) MXH_W1(Relu, relu)
MXH_W1(Recip, recip) MXH_W1(LogicalNot, logical_not) MXH_W1(Same, same)
MXH_W1(Sigmoid, sigmoid) MXH_W1(Tanh, tanh) MXH_W1(Gelu, gelu) MXH_W1(Sin, sin) MXH_W1(Cos, cos) MXH_W1(Tan, tan) MXH_W1(Ln, ln)
MXH_W1(Log10, log10) MXH_W1(Log2, log2) MXH_W1(Exp, exp) MXH_W1(Exp10, exp10) MXH_W1(Exp2, exp2) MXH_W1(Softplus, softplus)
MXH_W1C(Elu, elu)
MXH_W1C(AddScalar, add_scalar) MXH_W1C(SubScalar, sub_scalar) MXH_W1C(MulScalar, mul_scalar) MXH_W1C(DivScalar, div_scalar)
MXH_W1C(MaximumScalar, maximum_scalar) MXH_W1C(MinimumScalar, minimum_scalar) MXH_W1C(LeakyRelu, leaky_relu) MXH_W1C(Pow, pow)
// comparisons with a constant: on the value itself (bool: false < true), unary.rs:656-740
#define MXH_WCMP(NAME, SYM)                                                                    \
    template <class T> struct W##NAME {                                                        \
        using In = T; using Out = bool_t; static constexpr int NIN = 1;                        \
        T c;                                                                                   \
        __device__ bool_t operator()(T x) const { return (bool_t)(V(x) SYM V(c)); }            \
    };
MXH_WCMP(EqScalar, ==) MXH_WCMP(NeScalar, !=) MXH_WCMP(LtScalar, <) MXH_WCMP(LeScalar, <=) MXH_WCMP(GtScalar, >) MXH_WCMP(GeScalar, >=)

}  // namespace mxh

// P = the pointer / by-value type of the C ABI (uint8_t for bool), T the element type of the kernels
#define MXH_WU(NAME, OP, T, P, SUF, PO)                                                                        \
    extern "C" void hip_##NAME##_##SUF(size_t num_els, size_t num_dims, const size_t* md, const P* in, PO* out) { MXH_API; \
        using O = typename mxh::OP<T>::Out;                                                                    \
        mxh::ew_unary(num_els, num_dims, md, (const T*)in, (O*)out, mxh::OP<T>{});                             \
    }
#define MXH_WUC(NAME, OP, T, P, SUF, PO)                                                                       \
    extern "C" void hip_##NAME##_##SUF(size_t num_els, size_t num_dims, const size_t* md, const P* in, P c, PO* out) { MXH_API; \
        using O = typename mxh::OP<T>::Out;                                                                    \
        T ct;                                                                                                  \
        static_assert(sizeof(T) == sizeof(P), "ABI type and element type differ in size");                     \
        __builtin_memcpy(&ct, &c, sizeof(T));                                                                  \
        mxh::ew_unary(num_els, num_dims, md, (const T*)in, (O*)out, mxh::OP<T>{ct});                           \
    }
// the forms every one of these dtypes has
#define MXH_WIDE_COMMON(T, P, SUF)                                                                             \
    MXH_WU(logical_not, WLogicalNot, T, P, SUF, uint8_t)                                                       \
    MXH_WUC(add_scalar, WAddScalar, T, P, SUF, P) MXH_WUC(sub_scalar, WSubScalar, T, P, SUF, P)                \
    MXH_WUC(mul_scalar, WMulScalar, T, P, SUF, P) MXH_WUC(div_scalar, WDivScalar, T, P, SUF, P)                \
    MXH_WUC(maximum_scalar, WMaximumScalar, T, P, SUF, P) MXH_WUC(minimum_scalar, WMinimumScalar, T, P, SUF, P) \
    MXH_WUC(eq_scalar, WEqScalar, T, P, SUF, uint8_t) MXH_WUC(ne_scalar, WNeScalar, T, P, SUF, uint8_t)        \
    MXH_WUC(lt_scalar, WLtScalar, T, P, SUF, uint8_t) MXH_WUC(le_scalar, WLeScalar, T, P, SUF, uint8_t)        \
    MXH_WUC(gt_scalar, WGtScalar, T, P, SUF, uint8_t) MXH_WUC(ge_scalar, WGeScalar, T, P, SUF, uint8_t)
#define MXH_WIDE_UNSIGNED(T, SUF)                                                                              \
    MXH_WIDE_COMMON(T, T, SUF)                                                                                 \
    MXH_WU(sign, WSign, T, T, SUF, T) MXH_WU(square, WSquare, T, T, SUF, T) MXH_WU(sqrt, WSqrt, T, T, SUF, T)              \
    MXH_WUC(pow, WPow, T, T, SUF, T)
#define MXH_WIDE_SIGNED(T, SUF)                                                                                \
    MXH_WIDE_UNSIGNED(T, SUF) MXH_WU(neg, WNeg, T, T, SUF, T) MXH_WU(abs, WAbs, T, T, SUF, T)
