// Unary entry points for the unsigned integers (crates/maidenx_cuda/src/ops/unary.rs:105-120, 160-175).
#include "ops_wide.hpp"

MXH_WIDE_UNSIGNED(uint8_t, u8)
MXH_WIDE_UNSIGNED(uint16_t, u16)
MXH_WIDE_UNSIGNED(uint32_t, u32)
MXH_WIDE_UNSIGNED(uint64_t, u64)
