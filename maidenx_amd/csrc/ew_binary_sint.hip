// The binary families for the signed integers (crates/maidenx_cuda/src/ops/binary.rs:178-181): saturating
// arithmetic as in crates/maidenx_cpu/src/ops/binary.rs:379-382, 393-396, 407-410, 510-578.
#include "ew_binary.hpp"

MXH_ALL_FOR(int8_t, i8)
MXH_ALL_FOR(int16_t, i16)
MXH_ALL_FOR(int32_t, i32)
MXH_ALL_FOR(int64_t, i64)
