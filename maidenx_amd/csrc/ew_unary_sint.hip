// Unary entry points for the signed integers (crates/maidenx_cuda/src/ops/unary.rs:121-136, 176-191).
#include "ops_wide.hpp"

MXH_WIDE_SIGNED(int8_t, i8)
MXH_WIDE_SIGNED(int16_t, i16)
MXH_WIDE_SIGNED(int32_t, i32)
MXH_WIDE_SIGNED(int64_t, i64)
