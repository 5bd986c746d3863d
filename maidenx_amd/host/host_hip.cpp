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
    static void graph_begin() { if (hip_graph_begin_capture() != 0) throw mxt::Error(mxt::ErrKind::Backend, "hip_graph_begin_capture failed"); }
    static void graph_end(void** exec) { if (hip_graph_end_capture(exec) != 0) { *exec = nullptr; throw mxt::Error(mxt::ErrKind::Backend, "hip_graph_end_capture failed"); } }
    static void graph_launch(void* exec) { if (hip_graph_launch(exec) != 0) throw mxt::Error(mxt::ErrKind::Backend, "hip_graph_launch failed"); }
    static void graph_destroy(void* exec) { hip_graph_destroy(exec); }
    // host-side steps of the reference, done on the device
    static void fill_f32(size_t n, float* p, float v) { if (n) hip_fill_f32(n, p, v); }
    static void cast_bool_f32(size_t n, const uint8_t* in, float* out) { if (n) hip_cast_bool_f32(n, in, out); }
    static void copy_strided_f32(size_t n, size_t nd, const size_t* md, const float* in, float* out) { hip_copy_strided_f32(n, nd, md, in, out); }
    static void broadcast_scalar_f32(size_t n, const float* src, float* dst) {
        const size_t md[3] = {n, 0, 0};                    // dims [n], strides [0], offset 0
        hip_copy_strided_f32(n, 1, md, src, dst);
    }
    static constexpr auto add = &hip_add_f32;
    static constexpr auto sub = &hip_sub_f32;
    static constexpr auto mul = &hip_mul_f32;
    static constexpr auto div = &hip_div_f32;
    static constexpr auto add_inplace = &hip_add_inplace_f32;
    static constexpr auto sub_inplace = &hip_sub_inplace_f32;
    static constexpr auto neg = &hip_neg_f32;
    static constexpr auto square = &hip_square_f32;
    static constexpr auto relu = &hip_relu_f32;
    static constexpr auto tanh = &hip_tanh_f32;
    static constexpr auto gelu = &hip_gelu_f32;
    static constexpr auto exp = &hip_exp_f32;
    static constexpr auto add_scalar = &hip_add_scalar_f32;
    static constexpr auto mul_scalar = &hip_mul_scalar_f32;
    static constexpr auto div_scalar = &hip_div_scalar_f32;
    static constexpr auto pow = &hip_pow_f32;
    static constexpr auto gt_scalar = &hip_gt_scalar_f32;
    static constexpr auto sum = &hip_sum_f32;
    static constexpr auto mean = &hip_mean_f32;
    static constexpr auto sum_to_shape = &hip_sum_to_shape_f32;
    static constexpr auto matmul = &hip_matmul_f32;
    static constexpr auto matmul_backward = &hip_matmul_backward_f32;
    static constexpr auto im2col = &hip_conv2d_im2col_f32;
    static constexpr auto col2im = &hip_conv2d_col2im_f32;
};
using MxtBackend = HipBackend;
#include "mx_capi.hpp"
