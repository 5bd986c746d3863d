// Device-side fill, dtype conversion and strided copy.  The reference has no backend symbol
// for these: Tensor::fill / zeros / ones build a host vector and copy it
// (crates/maidenx_tensor/src/creation.rs:144-164), with_dtype converts on the host
// (crates/maidenx_core/src/buffer/mod.rs:155-196) and contiguous() copies element by element
// through get/set (crates/maidenx_tensor/src/f.rs:19-30).  A device backend needs them to keep
// a training step on the GPU.
#include "elementwise.hpp"
#include "ops.hpp"

namespace mxh {

template <class TI, class TO> struct OpConvert;
template <> struct OpConvert<bool_t, float> { using In = bool_t; using Out = float; static constexpr int NIN = 1;
    __device__ float operator()(bool_t x) const { return x ? 1.0f : 0.0f; } };
template <> struct OpConvert<bool_t, bf16_t> { using In = bool_t; using Out = bf16_t; static constexpr int NIN = 1;
    __device__ bf16_t operator()(bool_t x) const { return bf16_t{(uint16_t)(x ? 0x3F80 : 0)}; } };
template <> struct OpConvert<float, bf16_t> { using In = float; using Out = bf16_t; static constexpr int NIN = 1;
    __device__ bf16_t operator()(float x) const { return f2bf(x); } };
template <> struct OpConvert<bf16_t, float> { using In = bf16_t; using Out = float; static constexpr int NIN = 1;
    __device__ float operator()(bf16_t x) const { return bf2f(x); } };
template <> struct OpConvert<bool_t, f16_t> { using In = bool_t; using Out = f16_t; static constexpr int NIN = 1;
    __device__ f16_t operator()(bool_t x) const { return f16_t{(uint16_t)(x ? 0x3C00 : 0)}; } };
template <> struct OpConvert<float, f16_t> { using In = float; using Out = f16_t; static constexpr int NIN = 1;
    __device__ f16_t operator()(float x) const { return f2h(x); } };
template <> struct OpConvert<f16_t, float> { using In = f16_t; using Out = float; static constexpr int NIN = 1;
    __device__ float operator()(f16_t x) const { return h2f(x); } };
template <> struct OpConvert<f16_t, bool_t> { using In = f16_t; using Out = bool_t; static constexpr int NIN = 1;
    __device__ bool_t operator()(f16_t x) const { return (bool_t)(h2f(x) != 0.0f); } };
template <> struct OpConvert<float, bool_t> { using In = float; using Out = bool_t; static constexpr int NIN = 1;
    __device__ bool_t operator()(float x) const { return (bool_t)(x != 0.0f); } };
template <> struct OpConvert<bf16_t, bool_t> { using In = bf16_t; using Out = bool_t; static constexpr int NIN = 1;
    __device__ bool_t operator()(bf16_t x) const { return (bool_t)(bf2f(x) != 0.0f); } };

}  // namespace mxh

using namespace mxh;

#define MXH_UTIL_FOR(T, SUF)                                                                               \
    /* out[0..n) = value */                                                                                \
    extern "C" void hip_fill_##SUF(size_t n, T* out, T value) { MXH_API;                                   \
        ew_unary(n, 1, nullptr, nullptr, out, OpFill<T>{value});                                           \
    }                                                                                                      \
    /* contiguous copy of a strided view; metadata as for the unary ops: dims | strides | offset */        \
    extern "C" void hip_copy_strided_##SUF(size_t n, size_t nd, const size_t* md, const T* in, T* out) { MXH_API; \
        ew_unary(n, nd, md, in, out, OpIdentity<T>{});                                                     \
    }
MXH_UTIL_FOR(float, f32)
MXH_UTIL_FOR(bf16_t, bf16)
MXH_UTIL_FOR(f16_t, f16)
extern "C" void hip_fill_bool(size_t n, bool_t* out, bool_t value) { MXH_API; ew_unary(n, 1, nullptr, nullptr, out, OpFill<bool_t>{value}); }

#define MXH_CAST(TI, SI, TO, SO)                                                                           \
    extern "C" void hip_cast_##SI##_##SO(size_t n, const TI* in, TO* out) { MXH_API;                       \
        if (!in) { set_status(ERR_INVALID, "cast: null input"); return; }                                  \
        ew_unary(n, 1, nullptr, in, out, OpConvert<TI, TO>{});                                             \
    }
MXH_CAST(bool_t, bool, float, f32)
MXH_CAST(bool_t, bool, bf16_t, bf16)
MXH_CAST(float, f32, bf16_t, bf16)
MXH_CAST(bf16_t, bf16, float, f32)
MXH_CAST(bool_t, bool, f16_t, f16)
MXH_CAST(float, f32, f16_t, f16)
MXH_CAST(f16_t, f16, float, f32)
MXH_CAST(f16_t, f16, bool_t, bool)
MXH_CAST(float, f32, bool_t, bool)
MXH_CAST(bf16_t, bf16, bool_t, bool)
