// The binary families for the unsigned integers (crates/maidenx_cuda/src/ops/binary.rs:174-177): saturating
// arithmetic as in crates/maidenx_cpu/src/ops/binary.rs:375-378, 389-392, 403-406, 458-509.
#include "ew_binary.hpp"

MXH_ALL_FOR(uint8_t, u8)
MXH_ALL_FOR(uint16_t, u16)
MXH_ALL_FOR(uint32_t, u32)
MXH_ALL_FOR(uint64_t, u64)
