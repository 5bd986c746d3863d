// hip_cast_bool_<dtype>: device-side conversions from bool (the rules are stated in cast.hpp).
#include "cast.hpp"

MXH_CAST_WIDE(mxh::b8_t, uint8_t, bool, double, double, f64)
MXH_CAST_WIDE(mxh::b8_t, uint8_t, bool, uint8_t, uint8_t, u8)
MXH_CAST_WIDE(mxh::b8_t, uint8_t, bool, uint16_t, uint16_t, u16)
MXH_CAST_WIDE(mxh::b8_t, uint8_t, bool, uint32_t, uint32_t, u32)
MXH_CAST_WIDE(mxh::b8_t, uint8_t, bool, uint64_t, uint64_t, u64)
MXH_CAST_WIDE(mxh::b8_t, uint8_t, bool, int8_t, int8_t, i8)
MXH_CAST_WIDE(mxh::b8_t, uint8_t, bool, int16_t, int16_t, i16)
MXH_CAST_WIDE(mxh::b8_t, uint8_t, bool, int32_t, int32_t, i32)
MXH_CAST_WIDE(mxh::b8_t, uint8_t, bool, int64_t, int64_t, i64)
