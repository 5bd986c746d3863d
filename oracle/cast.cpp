// TEST INFRASTRUCTURE ONLY — CPU restatement of the reference's dtype conversion for the plain-number dtypes
// (crates/maidenx_core/src/buffer/mod.rs:155-196 with the pair table at :414-560): `x as T` between Rust primitives,
// `x != default` towards bool (:244-262), bool through u8 (:436-446).  Rust's `as` from a float to an integer drops the
// fraction, saturates at the target's bounds and sends NaN to 0; restated here in 80-bit long double, which holds every
// 64-bit integer exactly.
#include <cmath>
#include <cstddef>
#include <cstdint>
#include <limits>
#include <type_traits>

namespace {

template <class TO, class TI> inline TO convert(TI x) {
    if constexpr (std::is_same<TO, bool>::value) return x != TI(0);
    else if constexpr (std::is_same<TI, bool>::value) return (TO)(uint8_t)(x ? 1 : 0);
    else if constexpr (std::is_floating_point<TI>::value && std::is_integral<TO>::value) {
        if (std::isnan(x)) return 0;
        const long double t = std::trunc((long double)x);
        const long double lo = (long double)std::numeric_limits<TO>::min(), hi = (long double)std::numeric_limits<TO>::max();
        if (t < lo) return std::numeric_limits<TO>::min();
        if (t > hi) return std::numeric_limits<TO>::max();
        return (TO)t;
    } else return (TO)x;        // widening, narrowing (low bits kept) and integer -> float (round to nearest even)
}

}  // namespace

#define ORC_CAST(TI, SI, TO, SO)                                                     \
    extern "C" void oracle_cast_##SI##_##SO(size_t n, const TI* in, TO* out) {       \
        for (size_t i = 0; i < n; ++i) out[i] = convert<TO, TI>(in[i]);              \
    }
ORC_CAST(float, f32, double, f64)
ORC_CAST(float, f32, bool, bool)
ORC_CAST(float, f32, uint8_t, u8)
ORC_CAST(float, f32, uint16_t, u16)
ORC_CAST(float, f32, uint32_t, u32)
ORC_CAST(float, f32, uint64_t, u64)
ORC_CAST(float, f32, int8_t, i8)
ORC_CAST(float, f32, int16_t, i16)
ORC_CAST(float, f32, int32_t, i32)
ORC_CAST(float, f32, int64_t, i64)
ORC_CAST(double, f64, float, f32)
ORC_CAST(double, f64, bool, bool)
ORC_CAST(double, f64, uint8_t, u8)
ORC_CAST(double, f64, uint16_t, u16)
ORC_CAST(double, f64, uint32_t, u32)
ORC_CAST(double, f64, uint64_t, u64)
ORC_CAST(double, f64, int8_t, i8)
ORC_CAST(double, f64, int16_t, i16)
ORC_CAST(double, f64, int32_t, i32)
ORC_CAST(double, f64, int64_t, i64)
ORC_CAST(bool, bool, float, f32)
ORC_CAST(bool, bool, double, f64)
ORC_CAST(bool, bool, uint8_t, u8)
ORC_CAST(bool, bool, uint16_t, u16)
ORC_CAST(bool, bool, uint32_t, u32)
ORC_CAST(bool, bool, uint64_t, u64)
ORC_CAST(bool, bool, int8_t, i8)
ORC_CAST(bool, bool, int16_t, i16)
ORC_CAST(bool, bool, int32_t, i32)
ORC_CAST(bool, bool, int64_t, i64)
ORC_CAST(uint8_t, u8, float, f32)
ORC_CAST(uint8_t, u8, double, f64)
ORC_CAST(uint8_t, u8, bool, bool)
ORC_CAST(uint8_t, u8, uint16_t, u16)
ORC_CAST(uint8_t, u8, uint32_t, u32)
ORC_CAST(uint8_t, u8, uint64_t, u64)
ORC_CAST(uint8_t, u8, int8_t, i8)
ORC_CAST(uint8_t, u8, int16_t, i16)
ORC_CAST(uint8_t, u8, int32_t, i32)
ORC_CAST(uint8_t, u8, int64_t, i64)
ORC_CAST(uint16_t, u16, float, f32)
ORC_CAST(uint16_t, u16, double, f64)
ORC_CAST(uint16_t, u16, bool, bool)
ORC_CAST(uint16_t, u16, uint8_t, u8)
ORC_CAST(uint16_t, u16, uint32_t, u32)
ORC_CAST(uint16_t, u16, uint64_t, u64)
ORC_CAST(uint16_t, u16, int8_t, i8)
ORC_CAST(uint16_t, u16, int16_t, i16)
ORC_CAST(uint16_t, u16, int32_t, i32)
ORC_CAST(uint16_t, u16, int64_t, i64)
ORC_CAST(uint32_t, u32, float, f32)
ORC_CAST(uint32_t, u32, double, f64)
ORC_CAST(uint32_t, u32, bool, bool)
ORC_CAST(uint32_t, u32, uint8_t, u8)
ORC_CAST(uint32_t, u32, uint16_t, u16)
ORC_CAST(uint32_t, u32, uint64_t, u64)
ORC_CAST(uint32_t, u32, int8_t, i8)
ORC_CAST(uint32_t, u32, int16_t, i16)
ORC_CAST(uint32_t, u32, int32_t, i32)
ORC_CAST(uint32_t, u32, int64_t, i64)
ORC_CAST(uint64_t, u64, float, f32)
ORC_CAST(uint64_t, u64, double, f64)
ORC_CAST(uint64_t, u64, bool, bool)
ORC_CAST(uint64_t, u64, uint8_t, u8)
ORC_CAST(uint64_t, u64, uint16_t, u16)
ORC_CAST(uint64_t, u64, uint32_t, u32)
ORC_CAST(uint64_t, u64, int8_t, i8)
ORC_CAST(uint64_t, u64, int16_t, i16)
ORC_CAST(uint64_t, u64, int32_t, i32)
ORC_CAST(uint64_t, u64, int64_t, i64)
ORC_CAST(int8_t, i8, float, f32)
ORC_CAST(int8_t, i8, double, f64)
ORC_CAST(int8_t, i8, bool, bool)
ORC_CAST(int8_t, i8, uint8_t, u8)
ORC_CAST(int8_t, i8, uint16_t, u16)
ORC_CAST(int8_t, i8, uint32_t, u32)
ORC_CAST(int8_t, i8, uint64_t, u64)
ORC_CAST(int8_t, i8, int16_t, i16)
ORC_CAST(int8_t, i8, int32_t, i32)
ORC_CAST(int8_t, i8, int64_t, i64)
ORC_CAST(int16_t, i16, float, f32)
ORC_CAST(int16_t, i16, double, f64)
ORC_CAST(int16_t, i16, bool, bool)
ORC_CAST(int16_t, i16, uint8_t, u8)
ORC_CAST(int16_t, i16, uint16_t, u16)
ORC_CAST(int16_t, i16, uint32_t, u32)
ORC_CAST(int16_t, i16, uint64_t, u64)
ORC_CAST(int16_t, i16, int8_t, i8)
ORC_CAST(int16_t, i16, int32_t, i32)
ORC_CAST(int16_t, i16, int64_t, i64)
ORC_CAST(int32_t, i32, float, f32)
ORC_CAST(int32_t, i32, double, f64)
ORC_CAST(int32_t, i32, bool, bool)
ORC_CAST(int32_t, i32, uint8_t, u8)
ORC_CAST(int32_t, i32, uint16_t, u16)
ORC_CAST(int32_t, i32, uint32_t, u32)
ORC_CAST(int32_t, i32, uint64_t, u64)
ORC_CAST(int32_t, i32, int8_t, i8)
ORC_CAST(int32_t, i32, int16_t, i16)
ORC_CAST(int32_t, i32, int64_t, i64)
ORC_CAST(int64_t, i64, float, f32)
ORC_CAST(int64_t, i64, double, f64)
ORC_CAST(int64_t, i64, bool, bool)
ORC_CAST(int64_t, i64, uint8_t, u8)
ORC_CAST(int64_t, i64, uint16_t, u16)
ORC_CAST(int64_t, i64, uint32_t, u32)
ORC_CAST(int64_t, i64, uint64_t, u64)
ORC_CAST(int64_t, i64, int8_t, i8)
ORC_CAST(int64_t, i64, int16_t, i16)
ORC_CAST(int64_t, i64, int32_t, i32)
