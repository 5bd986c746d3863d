// TEST INFRASTRUCTURE ONLY. CPU restatement of the reference's maidenx_cpu crate.
// Nothing in the product (the HIP library, its host layer) may include, link or call
// this directory; only tests/, the smoke check and the cpu_baseline leg of bench.py do.
//
// Shared helpers: the bf16 storage type of the `half` crate (v2.6, a third-party
// dependency of the reference that is not vendored), the stride helpers of
// crates/maidenx_cpu/src/utils.rs, and the sequential / threaded execution switch.
#pragma once
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
struct bf16 {
    uint16_t bits;
    bf16() = default;
    static bf16 from_bits(uint16_t b) { bf16 r; r.bits = b; return r; }
    static bf16 from_f32(float f) {
        uint32_t x; std::memcpy(&x, &f, 4);
        if ((x & 0x7FFFFFFFu) > 0x7F800000u) return from_bits((uint16_t)((x >> 16) | 0x0040u));
        const uint32_t round_bit = 0x00008000u;
        if ((x & round_bit) != 0 && (x & (3u * round_bit - 1u)) != 0)
            return from_bits((uint16_t)((x >> 16) + 1u));
        return from_bits((uint16_t)(x >> 16));
    }
    float to_f32() const {
        uint32_t x = (uint32_t)bits << 16; float f; std::memcpy(&f, &x, 4); return f;
    }
};
inline bf16 operator+(bf16 a, bf16 b) { return bf16::from_f32(a.to_f32() + b.to_f32()); }
inline bf16 operator-(bf16 a, bf16 b) { return bf16::from_f32(a.to_f32() - b.to_f32()); }
inline bf16 operator*(bf16 a, bf16 b) { return bf16::from_f32(a.to_f32() * b.to_f32()); }
inline bf16 operator/(bf16 a, bf16 b) { return bf16::from_f32(a.to_f32() / b.to_f32()); }
inline bf16 operator-(bf16 a) { return bf16::from_bits((uint16_t)(a.bits ^ 0x8000u)); }
inline bf16& operator+=(bf16& a, bf16 b) { a = a + b; return a; }
inline bool operator==(bf16 a, bf16 b) { return a.to_f32() == b.to_f32(); }
inline bool operator!=(bf16 a, bf16 b) { return a.to_f32() != b.to_f32(); }
inline bool operator<(bf16 a, bf16 b) { return a.to_f32() < b.to_f32(); }
inline bool operator<=(bf16 a, bf16 b) { return a.to_f32() <= b.to_f32(); }
inline bool operator>(bf16 a, bf16 b) { return a.to_f32() > b.to_f32(); }
inline bool operator>=(bf16 a, bf16 b) { return a.to_f32() >= b.to_f32(); }

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

}  // namespace orc

#define ORC_PAR_FOR _Pragma("omp parallel for schedule(static) num_threads(orc::num_threads()) if (orc::num_threads() > 1)")
