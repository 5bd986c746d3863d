// extern "C" entry points of the binary, comparison, logical and in-place families: f32, bf16, f16.
#include "ew_binary.hpp"

MXH_ALL_FOR(float, f32)
MXH_ALL_FOR(bf16_t, bf16)
MXH_ALL_FOR(f16_t, f16)
