// TEST INFRASTRUCTURE ONLY — CPU restatement of crates/maidenx_cpu/src/ops/binary.rs.
// Symbols are the reference's `<op>_<dtype>` names with an `oracle_` prefix and the same
// argument order.  Metadata layout (binary.rs:39-51):
//   dims[n] | lhs_strides[n] | rhs_strides[n] | lhs_offset | rhs_offset
#include "common.hpp"

using namespace orc;

namespace {

struct Meta {
    const size_t *dims, *ls, *rs;
    size_t lo, ro;
    bool lc, rc;
};

// binary.rs:39-54 (and :152-173 for the in-place flavour): a null metadata pointer means
// "no dims": offsets 0 and both operands contiguous.
inline Meta parse(size_t num_dims, const size_t* md) {
    Meta m;
    if (md == nullptr) { m.dims = m.ls = m.rs = nullptr; m.lo = m.ro = 0; m.lc = m.rc = true; return m; }
    m.dims = md; m.ls = md + num_dims; m.rs = md + 2 * num_dims;
    m.lo = md[3 * num_dims]; m.ro = md[3 * num_dims + 1];
    m.lc = is_contiguous(num_dims, m.dims, m.ls);
    m.rc = is_contiguous(num_dims, m.dims, m.rs);
    return m;
}

// binary.rs:68-79: per-element walk from the last dim, skipping stride-0 dims.
inline size_t walk(size_t i, size_t num_dims, const size_t* dims, const size_t* strides) {
    size_t tmp = i, r = 0;
    for (size_t d = num_dims; d-- > 0;) {
        size_t i_dim = tmp % dims[d];
        r += strides[d] != 0 ? i_dim * strides[d] : 0;
        tmp /= dims[d];
    }
    return r;
}

// binary.rs:13-124 (binary_op_with_output!) — out is always written contiguously.
template <typename T, typename O, typename F>
void binary_out(size_t num_els, size_t num_dims, const size_t* md, const T* lhs, const T* rhs, O* out, F f) {
    Meta m = parse(num_dims, md);
    const T* l = lhs + m.lo;
    const T* r = rhs + m.ro;
    if (m.lc && m.rc) {
        ORC_PAR_FOR
        for (size_t i = 0; i < num_els; ++i) out[i] = (O)f(l[i], r[i]);
    } else if (m.lc) {
        ORC_PAR_FOR
        for (size_t i = 0; i < num_els; ++i) out[i] = (O)f(l[i], r[walk(i, num_dims, m.dims, m.rs)]);
    } else if (m.rc) {
        ORC_PAR_FOR
        for (size_t i = 0; i < num_els; ++i) out[i] = (O)f(l[walk(i, num_dims, m.dims, m.ls)], r[i]);
    } else {
        ORC_PAR_FOR
        for (size_t i = 0; i < num_els; ++i)
            out[i] = (O)f(l[walk(i, num_dims, m.dims, m.ls)], r[walk(i, num_dims, m.dims, m.rs)]);
    }
}

// binary.rs:126-248 (binary_op_inplace!) — serial on purpose, as in the reference.
template <typename T, typename F>
void binary_inplace(size_t num_els, size_t num_dims, const size_t* md, T* lhs, const T* rhs, F f) {
    Meta m = parse(num_dims, md);
    for (size_t i = 0; i < num_els; ++i) {
        size_t li = m.lc ? i : walk(i, num_dims, m.dims, m.ls);
        size_t ri = m.rc ? i : walk(i, num_dims, m.dims, m.rs);
        T* lv = lhs + m.lo + li;
        *lv = f(*lv, rhs[m.ro + ri]);
    }
}

// ---- element functions -----------------------------------------------------------------
template <typename T> inline T zero_of() { return T(0); }
template <> inline bf16 zero_of<bf16>() { return bf16::from_f32(0.0f); }
template <> inline f16 zero_of<f16>() { return f16::from_f32(0.0f); }
template <typename T> inline T inf_of() { return std::numeric_limits<T>::infinity(); }
template <> inline bf16 inf_of<bf16>() { return bf16::from_f32(std::numeric_limits<float>::infinity()); }
template <> inline f16 inf_of<f16>() { return f16::from_f32(std::numeric_limits<float>::infinity()); }

// Integers: Rust's saturating_add / _sub / _mul / _div (binary.rs:375-382, 389-396, 403-410, 458-578), restated as
// "compute exactly in 128 bits, clamp to the type".  bool (:374, 388, 402, 457): or, and, xor, and.
template <typename T> struct is_int : std::integral_constant<bool, std::is_integral<T>::value && !std::is_same<T, bool>::value> {};
template <typename T> using wide_t = typename std::conditional<std::is_signed<T>::value, __int128, unsigned __int128>::type;
template <typename T> inline T clamp_to(wide_t<T> v) {
    const wide_t<T> lo = std::numeric_limits<T>::min(), hi = std::numeric_limits<T>::max();
    return (T)(v < lo ? lo : (v > hi ? hi : v));
}

template <typename T> inline T op_add(T a, T b) {   // binary.rs:370-382
    if constexpr (std::is_same<T, bool>::value) return a | b;
    else if constexpr (is_int<T>::value) return clamp_to<T>((wide_t<T>)a + (wide_t<T>)b);
    else return a + b;
}
template <typename T> inline T op_sub(T a, T b) {   // binary.rs:384-396
    if constexpr (std::is_same<T, bool>::value) return a & b;
    else if constexpr (is_int<T>::value) {
        if (!std::is_signed<T>::value && b > a) return 0;           // (an unsigned difference below zero)
        return clamp_to<T>((wide_t<T>)a - (wide_t<T>)b);
    } else return a - b;
}
template <typename T> inline T op_mul(T a, T b) {   // binary.rs:398-410
    if constexpr (std::is_same<T, bool>::value) return a ^ b;
    else if constexpr (is_int<T>::value) {
        if (!std::is_signed<T>::value && sizeof(T) == 8) {          // the exact product of two u64 can exceed 128 signed bits but not 128 unsigned
            unsigned __int128 p = (unsigned __int128)a * (unsigned __int128)b;
            return p > (unsigned __int128)std::numeric_limits<T>::max() ? std::numeric_limits<T>::max() : (T)p;
        }
        return clamp_to<T>((wide_t<T>)a * (wide_t<T>)b);
    } else return a * b;
}
// binary.rs:412-465: b == 0 ⇒ (a == 0 ? 0 : +INF), sign of a ignored, NaN a ⇒ +INF.
// Integers (:458-578): b == 0 ⇒ 0 for a == 0, else MAX (MIN for a negative a); otherwise the quotient, clamped (MIN / -1).
template <typename T> inline T op_div(T a, T b) {
    if constexpr (std::is_same<T, bool>::value) return a & b;
    else if constexpr (is_int<T>::value) {
        if (b == 0) return a == 0 ? (T)0 : (a < 0 ? std::numeric_limits<T>::min() : std::numeric_limits<T>::max());
        return clamp_to<T>((wide_t<T>)a / (wide_t<T>)b);
    } else {
        if (b == zero_of<T>()) return a == zero_of<T>() ? zero_of<T>() : inf_of<T>();
        return a / b;
    }
}
// binary.rs:580-583: f32/f64 use `f32::max` (a NaN operand is ignored; fmax has that rule),
// bf16/f16 use `if a > b { a } else { b }`.
inline float op_maximum(float a, float b) { return std::fmax(a, b); }
inline double op_maximum(double a, double b) { return std::fmax(a, b); }
inline bf16 op_maximum(bf16 a, bf16 b) { return a > b ? a : b; }
inline f16 op_maximum(f16 a, f16 b) { return a > b ? a : b; }
inline float op_minimum(float a, float b) { return std::fmin(a, b); }   // binary.rs:594-597
inline double op_minimum(double a, double b) { return std::fmin(a, b); }
inline bf16 op_minimum(bf16 a, bf16 b) { return a < b ? a : b; }
inline f16 op_minimum(f16 a, f16 b) { return a < b ? a : b; }
// binary.rs:584-592, 598-606: bool or / and, integers Ord::max / Ord::min
template <typename T, typename = typename std::enable_if<std::is_integral<T>::value>::type> inline T op_maximum(T a, T b) {
    if constexpr (std::is_same<T, bool>::value) return a | b;
    else return a > b ? a : b;
}
template <typename T, typename = typename std::enable_if<std::is_integral<T>::value>::type> inline T op_minimum(T a, T b) {
    if constexpr (std::is_same<T, bool>::value) return a & b;
    else return a < b ? a : b;
}

}  // namespace

#define ORC_BINARY(NAME, T, SUF, FN)                                                                   \
    extern "C" void oracle_##NAME##_##SUF(size_t num_els, size_t num_dims, const size_t* md, const T* lhs, \
                                          const T* rhs, T* out) {                                      \
        binary_out<T, T>(num_els, num_dims, md, lhs, rhs, out, [](T a, T b) { return FN(a, b); });     \
    }
#define ORC_COMPARE(NAME, T, SUF, EXPR)                                                                \
    extern "C" void oracle_##NAME##_##SUF(size_t num_els, size_t num_dims, const size_t* md, const T* lhs, \
                                          const T* rhs, bool* out) {                                   \
        binary_out<T, bool>(num_els, num_dims, md, lhs, rhs, out, [](T a, T b) { return EXPR; });      \
    }
#define ORC_LOGICAL(NAME, T, SUF, EXPR)                                                                \
    extern "C" void oracle_##NAME##_##SUF(size_t num_els, size_t num_dims, const size_t* md, const T* lhs, \
                                          const T* rhs, bool* out) {                                   \
        binary_out<T, bool>(num_els, num_dims, md, lhs, rhs, out, [](T x, T y) {                       \
            bool a = x != zero_of<T>(), b = y != zero_of<T>();                                         \
            return EXPR;                                                                               \
        });                                                                                            \
    }
#define ORC_INPLACE(NAME, T, SUF, FN)                                                                  \
    extern "C" void oracle_##NAME##_inplace_##SUF(size_t num_els, size_t num_dims, const size_t* md, T* lhs, \
                                                  const T* rhs) {                                      \
        binary_inplace<T>(num_els, num_dims, md, lhs, rhs, [](T a, T b) { return FN(a, b); });         \
    }

#define ORC_ALL_FOR(T, SUF)                                   \
    ORC_BINARY(add, T, SUF, op_add<T>)                        \
    ORC_BINARY(sub, T, SUF, op_sub<T>)                        \
    ORC_BINARY(mul, T, SUF, op_mul<T>)                        \
    ORC_BINARY(div, T, SUF, op_div<T>)                        \
    ORC_BINARY(maximum, T, SUF, op_maximum)                   \
    ORC_BINARY(minimum, T, SUF, op_minimum)                   \
    /* binary.rs:250-368 (logical_op!): operands are first turned into `!= zero` */ \
    ORC_LOGICAL(logical_and, T, SUF, a && b)                  \
    ORC_LOGICAL(logical_or, T, SUF, a || b)                   \
    ORC_LOGICAL(logical_xor, T, SUF, a != b)                  \
    ORC_COMPARE(eq, T, SUF, a == b)                           \
    ORC_COMPARE(ne, T, SUF, a != b)                           \
    ORC_COMPARE(lt, T, SUF, a < b)                            \
    ORC_COMPARE(le, T, SUF, a <= b)                           \
    ORC_COMPARE(gt, T, SUF, a > b)                            \
    ORC_COMPARE(ge, T, SUF, a >= b)                           \
    ORC_INPLACE(add, T, SUF, op_add<T>)                       \
    ORC_INPLACE(sub, T, SUF, op_sub<T>)                       \
    ORC_INPLACE(mul, T, SUF, op_mul<T>)                       \
    ORC_INPLACE(div, T, SUF, op_div<T>)

ORC_ALL_FOR(float, f32)
ORC_ALL_FOR(double, f64)
ORC_ALL_FOR(bf16, bf16)
ORC_ALL_FOR(f16, f16)
ORC_ALL_FOR(bool, bool)
ORC_ALL_FOR(uint8_t, u8)
ORC_ALL_FOR(uint16_t, u16)
ORC_ALL_FOR(uint32_t, u32)
ORC_ALL_FOR(uint64_t, u64)
ORC_ALL_FOR(int8_t, i8)
ORC_ALL_FOR(int16_t, i16)
ORC_ALL_FOR(int32_t, i32)
ORC_ALL_FOR(int64_t, i64)
