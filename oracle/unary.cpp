// TEST INFRASTRUCTURE ONLY — CPU restatement of crates/maidenx_cpu/src/ops/unary.rs.
// Metadata layout (unary.rs:38-44):  dims[n] | strides[n] | offset
// Transcendentals go to the platform libm exactly as Rust's f32::exp/tanh/powf do
// (LLVM intrinsics lowered to expf/tanhf/powf); this file must be built with
// -ffp-contract=off so that no multiply-add is fused (Rust never contracts).
#include "common.hpp"

using namespace orc;

namespace {

// unary.rs:14-63 (unary_op_output!) and :71-122 (unary_op_with_constant_output!)
template <typename T, typename O, typename F>
void unary_out(size_t num_els, size_t num_dims, const size_t* md, const T* input, O* out, F f) {
    const size_t* dims = md;
    const size_t* strides = md ? md + num_dims : nullptr;
    size_t offset = md ? md[2 * num_dims] : 0;
    const T* inp = input + offset;
    if (md == nullptr || is_contiguous(num_dims, dims, strides)) {
        ORC_PAR_FOR
        for (size_t i = 0; i < num_els; ++i) out[i] = (O)f(inp[i]);
    } else {
        ORC_PAR_FOR
        for (size_t i = 0; i < num_els; ++i) out[i] = (O)f(inp[get_strided_index(i, num_dims, dims, strides)]);
    }
}

template <typename T> struct Fx;   // per-dtype element functions

template <typename R> struct FloatFx {   // R = float or double: everything in R, nothing fused
    using T = R;
    static T neg(T x) { return -x; }                                        // unary.rs:124
    static T abs(T x) { return std::fabs(x); }                              // :134
    static T sign(T x) { return x > 0 ? T(1) : (x < 0 ? T(-1) : T(0)); }    // :144-157
    static T square(T x) { return x * x; }                                  // :206
    static T sqrt(T x) { return std::sqrt(x); }                             // :220
    static T relu(T x) { return x > 0 ? x : T(0); }                         // :234  NaN→0, −0→+0
    static T sigmoid(T x) { return T(1) / (T(1) + std::exp(-x)); }          // :252
    static T tanh(T x) { return std::tanh(x); }                             // :262
    static T gelu(T x) {                                                    // :268-279
        const T sqrt_2_over_pi = (T)0.7978845608028654;
        const T coeff = (T)0.044715;
        T tanh_arg = sqrt_2_over_pi * (x + coeff * x * x * x);
        return (T)0.5 * x * (T(1) + std::tanh(tanh_arg));
    }
    static T sin(T x) { return std::sin(x); }
    static T cos(T x) { return std::cos(x); }
    static T tan(T x) { return std::tan(x); }
    static T ln(T x) { return std::log(x); }
    static T log10(T x) { return std::log10(x); }
    static T log2(T x) { return std::log2(x); }
    static T exp(T x) { return std::exp(x); }                               // :328
    static T exp10(T x) { return std::pow(T(10), x); }                      // :333
    static T exp2(T x) { return std::exp2(x); }
    static T softplus(T x) { return std::log(T(1) + std::exp(x)); }         // :343
    static T recip(T x) { return T(1) / x; }                                // :354
    static bool logical_not(T x) { return x == 0; }                         // :359
    static T add_scalar(T x, T c) { return x + c; }                         // :374
    static T sub_scalar(T x, T c) { return x - c; }
    static T mul_scalar(T x, T c) { return x * c; }                         // :402
    static T div_scalar(T x, T c) {                                         // :434-442
        if (c == 0) return x == 0 ? T(0) : std::numeric_limits<T>::infinity();
        return x / c;
    }
    static T maximum_scalar(T x, T c) { return std::fmax(x, c); }           // :536 f32::max
    static T minimum_scalar(T x, T c) { return std::fmin(x, c); }
    static T pow(T x, T c) { return std::pow(x, c); }                       // :562 powf even for c = 2
    static T leaky_relu(T x, T a) { return x > 0 ? x : a * x; }             // :580
    static T elu(T x, T a) { return x > 0 ? x : a * (std::exp(x) - T(1)); } // :605
    static bool eq_scalar(T x, T c) { return x == c; }
    static bool ne_scalar(T x, T c) { return x != c; }
    static bool lt_scalar(T x, T c) { return x < c; }
    static bool le_scalar(T x, T c) { return x <= c; }
    static bool gt_scalar(T x, T c) { return x > c; }
    static bool ge_scalar(T x, T c) { return x >= c; }
};
template <> struct Fx<float> : FloatFx<float> {};
template <> struct Fx<double> : FloatFx<double> {};

// bf16: "upcast, compute in f32, round once" for the transcendental forms, bf16 operators
// (round per op) for the arithmetic forms — each as written in unary.rs.
template <class C> struct Fx<half_t<C>> {
    using T = half_t<C>;
    using F = FloatFx<float>;
    static T r(float v) { return T::from_f32(v); }
    static T z() { return T::from_f32(0.0f); }
    static T neg(T x) { return -x; }                                        // :132 sign-bit flip
    static T abs(T x) { return r(std::fabs(x.to_f32())); }                  // :142
    static T sign(T x) { return x > z() ? r(1.0f) : (x < z() ? r(-1.0f) : z()); }
    static T square(T x) { return x * x; }                                  // :218
    static T sqrt(T x) { return r(std::sqrt(x.to_f32())); }
    static T relu(T x) { return x > z() ? x : z(); }                        // :244-250
    static T sigmoid(T x) { return r(1.0f / (1.0f + std::exp(-x.to_f32()))); }
    static T tanh(T x) { return r(std::tanh(x.to_f32())); }
    static T gelu(T x) { return r(F::gelu(x.to_f32())); }                   // :287-293
    static T sin(T x) { return r(std::sin(x.to_f32())); }
    static T cos(T x) { return r(std::cos(x.to_f32())); }
    static T tan(T x) { return r(std::tan(x.to_f32())); }
    static T ln(T x) { return r(std::log(x.to_f32())); }
    static T log10(T x) { return r(std::log10(x.to_f32())); }
    static T log2(T x) { return r(std::log2(x.to_f32())); }
    static T exp(T x) { return r(std::exp(x.to_f32())); }
    static T exp10(T x) { return r(std::pow(10.0f, x.to_f32())); }
    static T exp2(T x) { return r(std::exp2(x.to_f32())); }
    static T softplus(T x) { return r(std::log(1.0f + std::exp(x.to_f32()))); }
    static T recip(T x) { return r(1.0f / x.to_f32()); }
    static bool logical_not(T x) { return x == z(); }
    static T add_scalar(T x, T c) { return x + c; }
    static T sub_scalar(T x, T c) { return x - c; }
    static T mul_scalar(T x, T c) { return x * c; }
    static T div_scalar(T x, T c) {                                         // :416-424
        if (c == z()) return x == z() ? z() : r(std::numeric_limits<float>::infinity());
        return x / c;
    }
    static T maximum_scalar(T x, T c) { return x > c ? x : c; }             // :534
    static T minimum_scalar(T x, T c) { return x < c ? x : c; }
    static T pow(T x, T c) { return r(std::pow(x.to_f32(), c.to_f32())); }  // :576-578
    static T leaky_relu(T x, T a) { return x > z() ? x : a * x; }           // :597-603
    static T elu(T x, T a) {                                                // :628-636
        float xf = x.to_f32(), af = a.to_f32();
        return xf > 0.0f ? x : r(af * (std::exp(xf) - 1.0f));
    }
    static bool eq_scalar(T x, T c) { return x == c; }
    static bool ne_scalar(T x, T c) { return x != c; }
    static bool lt_scalar(T x, T c) { return x < c; }
    static bool le_scalar(T x, T c) { return x <= c; }
    static bool gt_scalar(T x, T c) { return x > c; }
    static bool ge_scalar(T x, T c) { return x >= c; }
};

// Integers (unary.rs:127-130, 137-140, 159-198, 209-216, 223-230, 362-369 and the scalar forms :377-384, 391-398,
// 405-412, 453-533, 539-560, 664-740).  Negation, absolute value and square overflow in the reference (a panic in a
// debug build, two's-complement wrap in a release build); the wrap is what is restated, through 128-bit arithmetic
// reduced modulo 2^bits.  The scalar add / sub / mul saturate.
template <typename I> struct IntFx {
    using T = I;
    using L = std::numeric_limits<I>;
    static T wrap(__int128 v) {                                   // v modulo 2^bits, as a T
        const __int128 span = (__int128)1 << (8 * sizeof(T));
        __int128 r = ((v % span) + span) % span;                  // 0 .. span-1
        if (std::is_signed<T>::value && r > (__int128)L::max()) r -= span;
        return (T)r;
    }
    static T sat(__int128 v) { return v < (__int128)L::min() ? L::min() : (v > (__int128)L::max() ? L::max() : (T)v); }
    static T neg(T x) { return wrap(-(__int128)x); }
    static T abs(T x) { return wrap(x < 0 ? -(__int128)x : (__int128)x); }
    static T sign(T x) { return x > 0 ? T(1) : (x < 0 ? T(-1) : T(0)); }
    static T square(T x) {
        if (!std::is_signed<T>::value && sizeof(T) == 8) return (T)((unsigned long long)x * (unsigned long long)x);   // (x^2 can pass 2^127: unsigned 64-bit product wraps as required)
        return wrap((__int128)x * (__int128)x);
    }
    static T sqrt(T x) {                                          // `(x as f32).sqrt() as T`; i64: f64; of |x| for signed types
        T a = std::is_signed<T>::value ? abs(x) : x;
        long double r = std::is_same<T, int64_t>::value ? (long double)std::sqrt((double)a) : (long double)std::sqrt((float)a);
        if (std::isnan(r)) return 0;
        r = std::trunc(r);
        return r > (long double)L::max() ? L::max() : (T)r;
    }
    // unary.rs:565-572: `(x as f64).powf(c as f64) as T` (u8 through f32), Rust's `as`: toward zero, saturating, NaN -> 0
    static T pow(T x, T c) {
        long double r = std::is_same<T, uint8_t>::value ? (long double)std::pow((float)x, (float)c) : (long double)std::pow((double)x, (double)c);
        if (std::isnan(r)) return 0;
        r = std::trunc(r);
        if (r >= (long double)L::max()) return L::max();
        if (r <= (long double)L::min()) return L::min();
        return (T)r;
    }
    static bool logical_not(T x) { return x == 0; }
    static T add_scalar(T x, T c) { return std::is_signed<T>::value || sizeof(T) < 8 ? sat((__int128)x + c) : (T)((unsigned __int128)x + c > L::max() ? L::max() : x + c); }
    static T sub_scalar(T x, T c) { return sat((__int128)x - (__int128)c); }
    static T mul_scalar(T x, T c) {
        if (!std::is_signed<T>::value && sizeof(T) == 8) {
            unsigned __int128 p = (unsigned __int128)x * (unsigned __int128)c;
            return p > (unsigned __int128)L::max() ? L::max() : (T)p;
        }
        return sat((__int128)x * (__int128)c);
    }
    static T div_scalar(T x, T c) {
        if (c == 0) return x == 0 ? T(0) : (x < 0 ? L::min() : L::max());
        if (!std::is_signed<T>::value) return x / c;
        return sat((__int128)x / (__int128)c);
    }
    static T maximum_scalar(T x, T c) { return x > c ? x : c; }
    static T minimum_scalar(T x, T c) { return x < c ? x : c; }
    static bool eq_scalar(T x, T c) { return x == c; }
    static bool ne_scalar(T x, T c) { return x != c; }
    static bool lt_scalar(T x, T c) { return x < c; }
    static bool le_scalar(T x, T c) { return x <= c; }
    static bool gt_scalar(T x, T c) { return x > c; }
    static bool ge_scalar(T x, T c) { return x >= c; }
};
template <> struct Fx<uint8_t> : IntFx<uint8_t> {};
template <> struct Fx<uint16_t> : IntFx<uint16_t> {};
template <> struct Fx<uint32_t> : IntFx<uint32_t> {};
template <> struct Fx<uint64_t> : IntFx<uint64_t> {};
template <> struct Fx<int8_t> : IntFx<int8_t> {};
template <> struct Fx<int16_t> : IntFx<int16_t> {};
template <> struct Fx<int32_t> : IntFx<int32_t> {};
template <> struct Fx<int64_t> : IntFx<int64_t> {};

// bool (unary.rs:126, 136, 158, 208, 222, 236, 254, 264, 361, 376, 390, 404, 452, 538, 552, 564, 656-661)
template <> struct Fx<bool> {
    using T = bool;
    static T neg(T x) { return !x; }
    static T abs(T x) { return x; }
    static T sign(T x) { return x; }
    static T square(T x) { return x; }
    static T sqrt(T x) { return x; }
    static T relu(T x) { return x; }
    static T sigmoid(T x) { return x; }
    static T tanh(T x) { return x; }
    static bool logical_not(T x) { return !x; }
    static T add_scalar(T x, T c) { return x || c; }
    static T sub_scalar(T x, T c) { return x ^ c; }
    static T mul_scalar(T x, T c) { return x && c; }
    static T div_scalar(T x, T c) { return x && c; }
    static T maximum_scalar(T x, T c) { return x | c; }
    static T minimum_scalar(T x, T c) { return x & c; }
    static T pow(T x, T) { return x; }
    static bool eq_scalar(T x, T c) { return x == c; }
    static bool ne_scalar(T x, T c) { return x != c; }
    static bool lt_scalar(T x, T c) { return (!x) && c; }
    static bool le_scalar(T x, T c) { return (!x) || c; }
    static bool gt_scalar(T x, T c) { return x && (!c); }
    static bool ge_scalar(T x, T c) { return x || (!c); }
};

}  // namespace

#define ORC_UNARY(NAME, T, SUF, O)                                                                    \
    extern "C" void oracle_##NAME##_##SUF(size_t num_els, size_t num_dims, const size_t* md, const T* in, O* out) { \
        unary_out<T, O>(num_els, num_dims, md, in, out, [](T x) { return Fx<T>::NAME(x); });          \
    }
#define ORC_UNARY_C(NAME, T, SUF, O)                                                                  \
    extern "C" void oracle_##NAME##_##SUF(size_t num_els, size_t num_dims, const size_t* md, const T* in, T c, O* out) { \
        unary_out<T, O>(num_els, num_dims, md, in, out, [c](T x) { return Fx<T>::NAME(x, c); });      \
    }

#define ORC_ALL_FOR(T, SUF)                                                                            \
    ORC_UNARY(neg, T, SUF, T) ORC_UNARY(abs, T, SUF, T) ORC_UNARY(sign, T, SUF, T)                     \
    ORC_UNARY(square, T, SUF, T) ORC_UNARY(sqrt, T, SUF, T) ORC_UNARY(relu, T, SUF, T)                 \
    ORC_UNARY(sigmoid, T, SUF, T) ORC_UNARY(tanh, T, SUF, T) ORC_UNARY(gelu, T, SUF, T)                \
    ORC_UNARY(sin, T, SUF, T) ORC_UNARY(cos, T, SUF, T) ORC_UNARY(tan, T, SUF, T)                      \
    ORC_UNARY(ln, T, SUF, T) ORC_UNARY(log10, T, SUF, T) ORC_UNARY(log2, T, SUF, T)                    \
    ORC_UNARY(exp, T, SUF, T) ORC_UNARY(exp10, T, SUF, T) ORC_UNARY(exp2, T, SUF, T)                   \
    ORC_UNARY(softplus, T, SUF, T) ORC_UNARY(recip, T, SUF, T) ORC_UNARY(logical_not, T, SUF, bool)    \
    ORC_UNARY_C(add_scalar, T, SUF, T) ORC_UNARY_C(sub_scalar, T, SUF, T)                              \
    ORC_UNARY_C(mul_scalar, T, SUF, T) ORC_UNARY_C(div_scalar, T, SUF, T)                              \
    ORC_UNARY_C(maximum_scalar, T, SUF, T) ORC_UNARY_C(minimum_scalar, T, SUF, T)                      \
    ORC_UNARY_C(pow, T, SUF, T) ORC_UNARY_C(leaky_relu, T, SUF, T) ORC_UNARY_C(elu, T, SUF, T)         \
    ORC_UNARY_C(eq_scalar, T, SUF, bool) ORC_UNARY_C(ne_scalar, T, SUF, bool)                          \
    ORC_UNARY_C(lt_scalar, T, SUF, bool) ORC_UNARY_C(le_scalar, T, SUF, bool)                          \
    ORC_UNARY_C(gt_scalar, T, SUF, bool) ORC_UNARY_C(ge_scalar, T, SUF, bool)

ORC_ALL_FOR(float, f32)
ORC_ALL_FOR(double, f64)
ORC_ALL_FOR(bf16, bf16)
ORC_ALL_FOR(f16, f16)

#define ORC_COMMON_FOR(T, SUF)                                                                         \
    ORC_UNARY(logical_not, T, SUF, bool)                                                               \
    ORC_UNARY_C(add_scalar, T, SUF, T) ORC_UNARY_C(sub_scalar, T, SUF, T)                              \
    ORC_UNARY_C(mul_scalar, T, SUF, T) ORC_UNARY_C(div_scalar, T, SUF, T)                              \
    ORC_UNARY_C(maximum_scalar, T, SUF, T) ORC_UNARY_C(minimum_scalar, T, SUF, T)                      \
    ORC_UNARY_C(eq_scalar, T, SUF, bool) ORC_UNARY_C(ne_scalar, T, SUF, bool)                          \
    ORC_UNARY_C(lt_scalar, T, SUF, bool) ORC_UNARY_C(le_scalar, T, SUF, bool)                          \
    ORC_UNARY_C(gt_scalar, T, SUF, bool) ORC_UNARY_C(ge_scalar, T, SUF, bool)
#define ORC_UNSIGNED_FOR(T, SUF)                                                                       \
    ORC_COMMON_FOR(T, SUF) ORC_UNARY(sign, T, SUF, T) ORC_UNARY(square, T, SUF, T) ORC_UNARY(sqrt, T, SUF, T) ORC_UNARY_C(pow, T, SUF, T)
#define ORC_SIGNED_FOR(T, SUF) ORC_UNSIGNED_FOR(T, SUF) ORC_UNARY(neg, T, SUF, T) ORC_UNARY(abs, T, SUF, T)

ORC_UNSIGNED_FOR(uint8_t, u8)
ORC_UNSIGNED_FOR(uint16_t, u16)
ORC_UNSIGNED_FOR(uint32_t, u32)
ORC_UNSIGNED_FOR(uint64_t, u64)
ORC_SIGNED_FOR(int8_t, i8)
ORC_SIGNED_FOR(int16_t, i16)
ORC_SIGNED_FOR(int32_t, i32)
ORC_SIGNED_FOR(int64_t, i64)
ORC_COMMON_FOR(bool, bool)
ORC_UNARY(neg, bool, bool, bool) ORC_UNARY(abs, bool, bool, bool) ORC_UNARY(sign, bool, bool, bool)
ORC_UNARY(square, bool, bool, bool) ORC_UNARY(sqrt, bool, bool, bool) ORC_UNARY(relu, bool, bool, bool)
ORC_UNARY(sigmoid, bool, bool, bool) ORC_UNARY(tanh, bool, bool, bool) ORC_UNARY_C(pow, bool, bool, bool)
