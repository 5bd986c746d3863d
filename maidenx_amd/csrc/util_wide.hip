// hip_fill_<dtype> / hip_copy_strided_<dtype> for f64, the integers and (copy) bool: the same kernels as for f32
// (util.hip), which has the reference lines these replace.
#include "elementwise.hpp"
#include "ops.hpp"

using namespace mxh;

#define MXH_UTIL_WIDE(T, SUF)                                                                              \
    extern "C" void hip_fill_##SUF(size_t n, T* out, T value) { MXH_API;                                   \
        ew_unary(n, 1, nullptr, nullptr, out, OpFill<T>{value});                                           \
    }                                                                                                      \
    extern "C" void hip_copy_strided_##SUF(size_t n, size_t nd, const size_t* md, const T* in, T* out) { MXH_API; \
        ew_unary(n, nd, md, in, out, OpIdentity<T>{});                                                     \
    }
MXH_UTIL_WIDE(double, f64)
MXH_UTIL_WIDE(uint8_t, u8)
MXH_UTIL_WIDE(uint16_t, u16)
MXH_UTIL_WIDE(uint32_t, u32)
MXH_UTIL_WIDE(uint64_t, u64)
MXH_UTIL_WIDE(int8_t, i8)
MXH_UTIL_WIDE(int16_t, i16)
MXH_UTIL_WIDE(int32_t, i32)
MXH_UTIL_WIDE(int64_t, i64)
extern "C" void hip_copy_strided_bool(size_t n, size_t nd, const size_t* md, const bool_t* in, bool_t* out) { MXH_API;
    ew_unary(n, nd, md, in, out, OpIdentity<bool_t>{});
}
