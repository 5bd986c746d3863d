// The binary families for f64 and bool (crates/maidenx_cuda/src/ops/binary.rs:172-173; element functions:
// crates/maidenx_cpu/src/ops/binary.rs:373-374 and the like).  `bool` buffers are bytes holding 0 or 1.
#include "ew_binary.hpp"

MXH_ALL_FOR(double, f64)
MXH_ALL_FOR(b8_t, bool)
