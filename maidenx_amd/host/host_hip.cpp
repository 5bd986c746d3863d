// libmaidenx_host.so: the host layer (mx_tensor.hpp) over the HIP backend's C ABI.
#include <string>

#include "../../include/maidenx_hip.h"
#include "mx_tensor.hpp"

struct HipBackend {
    static constexpr const char* name = "hip";
    static void* alloc(size_t bytes) {
        void* p = nullptr;
        return hip_malloc(&p, bytes) == 0 ? p : nullptr;
    }
    static void free(void* p) { hip_free(p); }
    static void sync() { hip_synchronize(); }
    static void h2d(void* d, const void* s, size_t n) { if (hip_memcpy_h2d(d, s, n) != 0) throw mxt::Error(mxt::ErrKind::Backend, "hip_memcpy_h2d failed"); }
    static void d2h(void* d, const void* s, size_t n) { if (hip_memcpy_d2h(d, s, n) != 0) throw mxt::Error(mxt::ErrKind::Backend, "hip_memcpy_d2h failed"); }
    static void check() {
        int st = hip_get_last_status();
        if (st != MX_HIP_OK) throw mxt::Error(st == MX_HIP_ERR_OOM ? mxt::ErrKind::OutOfMemory : mxt::ErrKind::Backend,
                                              std::string("HIP backend: ") + hip_status_string());
    }
    static constexpr bool has_graphs = true;
    static constexpr bool has_fused_adam = true;
    static constexpr bool has_fused_nn = true;
    static constexpr auto mse_loss = &hip_mse_loss_f32;
    static constexpr auto mse_loss_backward = &hip_mse_loss_backward_f32;
    static constexpr auto sgd_step = &hip_sgd_step_f32;
    static constexpr bool has_cols_matmul = true;
    static constexpr auto cols_matmul = &hip_conv2d_cols_matmul_f32;
    static constexpr bool has_col2im_add = true;
    static constexpr auto col2im_add = &hip_conv2d_col2im_add_f32;
    static constexpr bool has_conv_forward_product = true;
    static constexpr auto conv_forward_product = &hip_conv2d_forward_product_f32;
    static void graph_begin() { if (hip_graph_begin_capture() != 0) throw mxt::Error(mxt::ErrKind::Backend, "hip_graph_begin_capture failed"); }
    static void graph_end(void** exec) { if (hip_graph_end_capture(exec) != 0) { *exec = nullptr; throw mxt::Error(mxt::ErrKind::Backend, "hip_graph_end_capture failed"); } }
    static void graph_launch(void* exec) { if (hip_graph_launch(exec) != 0) throw mxt::Error(mxt::ErrKind::Backend, "hip_graph_launch failed"); }
    static void graph_launch_n(void* exec, size_t times) { if (hip_graph_launch_n(exec, times) != 0) throw mxt::Error(mxt::ErrKind::Backend, "hip_graph_launch_n failed"); }
    static void graph_destroy(void* exec) { hip_graph_destroy(exec); }
    static void discard(void* p, size_t bytes) { hip_buffer_discard(p, bytes); }
    // f32-only kernels (conv) and the float <-> float conversions
    static constexpr auto im2col = &hip_conv2d_im2col_f32;
    static constexpr auto col2im = &hip_conv2d_col2im_f32;
    static void cast_bf16_f32(size_t n, const uint16_t* in, float* out) { if (n) hip_cast_bf16_f32(n, in, out); }
    static void cast_f32_bf16(size_t n, const float* in, uint16_t* out) { if (n) hip_cast_f32_bf16(n, in, out); }
    // kernels per element type: float, and uint16_t holding bf16 bits
    template <class E> struct K;
};
#define MXT_HIP_KERNELS(E, S)                                                                                          \
    template <> struct HipBackend::K<E> {                                                                                \
        using Bin = void (*)(size_t, size_t, const size_t*, const E*, const E*, E*);                                     \
        using Inp = void (*)(size_t, size_t, const size_t*, E*, const E*);                                               \
        using Un = void (*)(size_t, size_t, const size_t*, const E*, E*);                                                \
        using Unc = void (*)(size_t, size_t, const size_t*, const E*, E, E*);                                            \
        using Red = void (*)(size_t, size_t, size_t, const size_t*, const E*, E*);                                       \
        static constexpr Bin bin[4] = {&hip_add_##S, &hip_sub_##S, &hip_mul_##S, &hip_div_##S};                          \
        static constexpr Inp inplace[2] = {&hip_add_inplace_##S, &hip_sub_inplace_##S};                                  \
        static constexpr Un un[7] = {&hip_neg_##S, &hip_square_##S, &hip_relu_##S, &hip_tanh_##S, &hip_gelu_##S, &hip_exp_##S, &hip_sqrt_##S}; \
        static constexpr Unc unc[4] = {&hip_add_scalar_##S, &hip_mul_scalar_##S, &hip_div_scalar_##S, &hip_pow_##S};      \
        static constexpr Red red[2] = {&hip_sum_##S, &hip_mean_##S};                                                     \
        static constexpr auto gt_scalar = &hip_gt_scalar_##S;                                                            \
        static constexpr auto sum_to_shape = &hip_sum_to_shape_##S;                                                      \
        static constexpr auto matmul = &hip_matmul_##S;                                                                  \
        static constexpr auto matmul_backward = &hip_matmul_backward_##S;                                                \
        static constexpr auto adam_step = &hip_adam_step_##S;                                                            \
        /* host-side steps of the reference, done on the device */                                                       \
        static void fill(size_t n, E* p, E v) { if (n) hip_fill_##S(n, p, v); }                                          \
        static void cast_from_bool(size_t n, const uint8_t* in, E* out) { if (n) hip_cast_bool_##S(n, in, out); }        \
        static void copy_strided(size_t n, size_t nd, const size_t* md, const E* in, E* out) { hip_copy_strided_##S(n, nd, md, in, out); } \
        static void broadcast_scalar(size_t n, const E* src, E* dst) {                                                   \
            const size_t md[3] = {n, 0, 0}; /* dims [n], strides [0], offset 0 */                                        \
            hip_copy_strided_##S(n, 1, md, src, dst);                                                                    \
        }                                                                                                                \
    };
MXT_HIP_KERNELS(float, f32)
MXT_HIP_KERNELS(uint16_t, bf16)
using MxtBackend = HipBackend;
#include "mx_capi.hpp"
