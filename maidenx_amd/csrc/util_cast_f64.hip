// hip_cast_f64_<dtype>: device-side conversions from f64 (the rules are stated in cast.hpp).
#include "cast.hpp"

MXH_CAST_WIDE(double, double, f64, float, float, f32)
MXH_CAST_WIDE(double, double, f64, mxh::b8_t, uint8_t, bool)
MXH_CAST_WIDE(double, double, f64, uint8_t, uint8_t, u8)
MXH_CAST_WIDE(double, double, f64, uint16_t, uint16_t, u16)
MXH_CAST_WIDE(double, double, f64, uint32_t, uint32_t, u32)
MXH_CAST_WIDE(double, double, f64, uint64_t, uint64_t, u64)
MXH_CAST_WIDE(double, double, f64, int8_t, int8_t, i8)
MXH_CAST_WIDE(double, double, f64, int16_t, int16_t, i16)
MXH_CAST_WIDE(double, double, f64, int32_t, int32_t, i32)
MXH_CAST_WIDE(double, double, f64, int64_t, int64_t, i64)
