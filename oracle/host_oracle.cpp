// TEST INFRASTRUCTURE ONLY.  The host layer of the product (maidenx_amd/host/mx_tensor.hpp) instantiated
// over the CPU oracle, so that tests can run the same tensor / autograd / nn programs on both backends and
// compare.  Built into oracle/liboracle_host.so; exports the C ABI of include/maidenx_host.h.
#include <cstdlib>
#include <cstring>

#include "../maidenx_amd/host/mx_tensor.hpp"

extern "C" {
#define ORC_BIN(N) void oracle_##N##_f32(size_t, size_t, const size_t*, const float*, const float*, float*);
ORC_BIN(add) ORC_BIN(sub) ORC_BIN(mul) ORC_BIN(div)
void oracle_add_inplace_f32(size_t, size_t, const size_t*, float*, const float*);
void oracle_sub_inplace_f32(size_t, size_t, const size_t*, float*, const float*);
#define ORC_UN(N) void oracle_##N##_f32(size_t, size_t, const size_t*, const float*, float*);
ORC_UN(neg) ORC_UN(square) ORC_UN(relu) ORC_UN(tanh) ORC_UN(gelu) ORC_UN(exp)
#define ORC_UNC(N) void oracle_##N##_f32(size_t, size_t, const size_t*, const float*, float, float*);
ORC_UNC(add_scalar) ORC_UNC(mul_scalar) ORC_UNC(div_scalar) ORC_UNC(pow)
void oracle_gt_scalar_f32(size_t, size_t, const size_t*, const float*, float, uint8_t*);
void oracle_sum_f32(size_t, size_t, size_t, const size_t*, const float*, float*);
void oracle_mean_f32(size_t, size_t, size_t, const size_t*, const float*, float*);
void oracle_sum_to_shape_f32(size_t, size_t, const size_t*, const float*, float*);
void oracle_matmul_f32(size_t, const size_t*, const float*, const float*, float*);
void oracle_matmul_backward_f32(size_t, size_t, const size_t*, const float*, const float*, const float*, float*, float*);
void oracle_conv2d_im2col_f32(size_t, const size_t*, const float*, float*);
void oracle_conv2d_col2im_f32(size_t, const size_t*, const float*, float*);
}

struct OracleBackend {
    static constexpr const char* name = "oracle";
    static void* alloc(size_t bytes) { return std::malloc(bytes); }
    static void free(void* p) { std::free(p); }
    static void sync() {}
    static void h2d(void* d, const void* s, size_t n) { std::memcpy(d, s, n); }
    static void d2h(void* d, const void* s, size_t n) { std::memcpy(d, s, n); }
    static void check() {}
    static constexpr bool has_graphs = false;
    // The reference does these on the host as well.
    static void fill_f32(size_t n, float* p, float v) { for (size_t i = 0; i < n; ++i) p[i] = v; }              // creation.rs:144-164, 253-305
    static void cast_bool_f32(size_t n, const uint8_t* in, float* out) { for (size_t i = 0; i < n; ++i) out[i] = in[i] ? 1.0f : 0.0f; }
    // crates/maidenx_tensor/src/f.rs:19-24: element by element through the logical index
    static void copy_strided_f32(size_t n, size_t nd, const size_t* md, const float* in, float* out) {
        const size_t *dims = md, *strides = md + nd;
        const size_t off = md[2 * nd];
        for (size_t i = 0; i < n; ++i) {
            size_t rem = i, src = off;
            for (size_t d = nd; d-- > 0;) {
                src += (rem % dims[d]) * strides[d];
                rem /= dims[d];
            }
            out[i] = in[src];
        }
    }
    static void broadcast_scalar_f32(size_t n, const float* src, float* dst) { fill_f32(n, dst, *src); }        // transform.rs:328-331
    static constexpr auto add = &oracle_add_f32;
    static constexpr auto sub = &oracle_sub_f32;
    static constexpr auto mul = &oracle_mul_f32;
    static constexpr auto div = &oracle_div_f32;
    static constexpr auto add_inplace = &oracle_add_inplace_f32;
    static constexpr auto sub_inplace = &oracle_sub_inplace_f32;
    static constexpr auto neg = &oracle_neg_f32;
    static constexpr auto square = &oracle_square_f32;
    static constexpr auto relu = &oracle_relu_f32;
    static constexpr auto tanh = &oracle_tanh_f32;
    static constexpr auto gelu = &oracle_gelu_f32;
    static constexpr auto exp = &oracle_exp_f32;
    static constexpr auto add_scalar = &oracle_add_scalar_f32;
    static constexpr auto mul_scalar = &oracle_mul_scalar_f32;
    static constexpr auto div_scalar = &oracle_div_scalar_f32;
    static constexpr auto pow = &oracle_pow_f32;
    static constexpr auto gt_scalar = &oracle_gt_scalar_f32;
    static constexpr auto sum = &oracle_sum_f32;
    static constexpr auto mean = &oracle_mean_f32;
    static constexpr auto sum_to_shape = &oracle_sum_to_shape_f32;
    static constexpr auto matmul = &oracle_matmul_f32;
    static constexpr auto matmul_backward = &oracle_matmul_backward_f32;
    static constexpr auto im2col = &oracle_conv2d_im2col_f32;
    static constexpr auto col2im = &oracle_conv2d_col2im_f32;
};
using MxtBackend = OracleBackend;
#include "../maidenx_amd/host/mx_capi.hpp"
