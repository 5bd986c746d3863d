// TEST INFRASTRUCTURE ONLY. CPU restatement of the reference's maidenx_cpu crate.
// Nothing in the product (the HIP library, its host layer) may include, link or call
// this directory; only tests/, the smoke check and the cpu_baseline leg of bench.py do.
//
// Shared helpers: the bf16 storage type of the `half` crate (v2.6, a third-party
// dependency of the reference that is not vendored), the stride helpers of
// crates/maidenx_cpu/src/utils.rs, and the sequential / threaded execution switch.
#pragma once
#include <type_traits>
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <limits>
#include <vector>

namespace orc {

// ---------------------------------------------------------------------------------------
// bf16 as the `half` crate defines it: 16 high bits of an IEEE-754 binary32, conversion
// from f32 by round-to-nearest-even on the dropped 16 bits, NaN kept NaN by forcing the
// quiet bit.  Arithmetic is "convert both to f32, operate, convert back" per operation
// (crates/maidenx_cpu/src/ops/binary.rs:372,400,416 use bf16 `+ - * /` directly).
// ---------------------------------------------------------------------------------------
// One 16-bit storage float = a codec (f32 <-> 16 bits) plus "convert, operate in f32, convert back"
// operators; bf16 and f16 differ only in the codec.
template <class Codec> struct half_t {
    uint16_t bits;
    half_t() = default;
    static half_t from_bits(uint16_t b) { half_t r; r.bits = b; return r; }
    static half_t from_f32(float f) { return from_bits(Codec::encode(f)); }
    float to_f32() const { return Codec::decode(bits); }
};
struct Bf16Codec {
    static uint16_t encode(float f) {
        uint32_t x; std::memcpy(&x, &f, 4);
        if ((x & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((x >> 16) | 0x0040u);
        const uint32_t round_bit = 0x00008000u;
        if ((x & round_bit) != 0 && (x & (3u * round_bit - 1u)) != 0) return (uint16_t)((x >> 16) + 1u);
        return (uint16_t)(x >> 16);
    }
    static float decode(uint16_t b) { uint32_t x = (uint32_t)b << 16; float f; std::memcpy(&f, &x, 4); return f; }
};
// IEEE binary16 (`half::f16`): 1 sign, 5 exponent (bias 15), 10 mantissa bits; round to nearest even,
// overflow to infinity, gradual underflow, NaN kept NaN with the quiet bit forced.
struct F16Codec {
    static uint16_t encode(float f) {
        uint32_t x; std::memcpy(&x, &f, 4);
        const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
        const uint32_t e = (x >> 23) & 0xFFu, m = x & 0x007FFFFFu;
        if (e == 0xFFu) return (uint16_t)(sign | 0x7C00u | (m ? 0x0200u : 0u) | (m >> 13));
        const int he = (int)e - 127 + 15;                    // exponent field of the half
        if (he >= 31) return (uint16_t)(sign | 0x7C00u);
        if (he <= 0) {                                       // subnormal half (or zero): shift the 24-bit significand
            if (he < -10) return sign;                       // below half of the smallest subnormal
            const uint32_t sig = m | 0x00800000u;
            const int shift = 14 - he;                       // 14 .. 24
            uint32_t hm = sig >> shift;
            const uint32_t rem = sig & ((1u << shift) - 1u), half = 1u << (shift - 1);
            if (rem > half || (rem == half && (hm & 1u))) ++hm;
            return (uint16_t)(sign | hm);                    // a carry into bit 10 is the smallest normal, as it should be
        }
        uint32_t h = ((uint32_t)he << 10) | (m >> 13);
        const uint32_t rem = m & 0x1FFFu;
        if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) ++h;      // a carry may reach the exponent: next binade or infinity
        return (uint16_t)(sign | h);
    }
    static float decode(uint16_t b) {
        const uint32_t sign = (uint32_t)(b & 0x8000u) << 16;
        uint32_t e = (b >> 10) & 0x1Fu, m = b & 0x3FFu, x;
        if (e == 0x1Fu) x = sign | 0x7F800000u | (m << 13);
        else if (e != 0) x = sign | ((e + 112u) << 23) | (m << 13);
        else if (m == 0) x = sign;
        else {                                               // subnormal: normalise
            int k = 0;
            while (!(m & 0x400u)) { m <<= 1; ++k; }
            x = sign | ((uint32_t)(113 - k) << 23) | ((m & 0x3FFu) << 13);
        }
        float f; std::memcpy(&f, &x, 4); return f;
    }
};
using bf16 = half_t<Bf16Codec>;
using f16 = half_t<F16Codec>;
template <class C> inline half_t<C> operator+(half_t<C> a, half_t<C> b) { return half_t<C>::from_f32(a.to_f32() + b.to_f32()); }
template <class C> inline half_t<C> operator-(half_t<C> a, half_t<C> b) { return half_t<C>::from_f32(a.to_f32() - b.to_f32()); }
template <class C> inline half_t<C> operator*(half_t<C> a, half_t<C> b) { return half_t<C>::from_f32(a.to_f32() * b.to_f32()); }
template <class C> inline half_t<C> operator/(half_t<C> a, half_t<C> b) { return half_t<C>::from_f32(a.to_f32() / b.to_f32()); }
template <class C> inline half_t<C> operator-(half_t<C> a) { return half_t<C>::from_bits((uint16_t)(a.bits ^ 0x8000u)); }
template <class C> inline half_t<C>& operator+=(half_t<C>& a, half_t<C> b) { a = a + b; return a; }
template <class C> inline bool operator==(half_t<C> a, half_t<C> b) { return a.to_f32() == b.to_f32(); }
template <class C> inline bool operator!=(half_t<C> a, half_t<C> b) { return a.to_f32() != b.to_f32(); }
template <class C> inline bool operator<(half_t<C> a, half_t<C> b) { return a.to_f32() < b.to_f32(); }
template <class C> inline bool operator<=(half_t<C> a, half_t<C> b) { return a.to_f32() <= b.to_f32(); }
template <class C> inline bool operator>(half_t<C> a, half_t<C> b) { return a.to_f32() > b.to_f32(); }
template <class C> inline bool operator>=(half_t<C> a, half_t<C> b) { return a.to_f32() >= b.to_f32(); }

// ---------------------------------------------------------------------------------------
// crates/maidenx_cpu/src/utils.rs:2-12  — contiguity test that ignores size-1 dims.
// ---------------------------------------------------------------------------------------
inline bool is_contiguous(size_t num_dims, const size_t* dims, const size_t* strides) {
    size_t acc = 1;
    for (size_t d = 0; d < num_dims; ++d) {
        size_t dim_idx = num_dims - 1 - d;
        if (dims[dim_idx] > 1 && acc != strides[dim_idx]) return false;
        acc *= dims[dim_idx];
    }
    return true;
}

// crates/maidenx_cpu/src/utils.rs:14-31 — logical index → memory index; stride-0 dims skipped.
inline size_t get_strided_index(size_t idx, size_t num_dims, const size_t* dims, const size_t* strides) {
    size_t strided_i = 0, remaining = idx;
    for (size_t d = 0; d < num_dims; ++d) {
        size_t dim_idx = num_dims - 1 - d;
        if (strides[dim_idx] != 0) strided_i += (remaining % dims[dim_idx]) * strides[dim_idx];
        remaining /= dims[dim_idx];
    }
    return strided_i;
}

// Number of worker threads: 1 = sequential, deterministic order (used for parity);
// >1 = the reference's rayon decomposition replayed with OpenMP (used for timing only).
int num_threads();

// `+=` of the reference's accumulating loops.  For the integer dtypes an overflow panics in the reference's debug build
// and wraps in its release build; the wrap is restated (through the unsigned type, where C++ defines it).
template <typename T> inline T add_wrap(T a, T b) {
    if constexpr (std::is_integral<T>::value) {
        using U = typename std::make_unsigned<T>::type;
        return (T)(U)((U)a + (U)b);
    } else return a + b;
}

}  // namespace orc

#define ORC_PAR_FOR _Pragma("omp parallel for schedule(static) num_threads(orc::num_threads()) if (orc::num_threads() > 1)")
