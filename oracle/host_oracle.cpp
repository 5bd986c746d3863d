// TEST INFRASTRUCTURE ONLY.  The host layer of the product (maidenx_amd/host/mx_tensor.hpp) instantiated
// over the CPU oracle, so that tests can run the same tensor / autograd / nn programs on both backends and
// compare.  Built into oracle/liboracle_host.so; exports the C ABI of include/maidenx_host.h.
#include <cstdlib>
#include <cstring>

#include "../maidenx_amd/host/mx_tensor.hpp"

extern "C" {
#define ORC_DECL(E, S)                                                                                             \
    void oracle_add_##S(size_t, size_t, const size_t*, const E*, const E*, E*);                                     \
    void oracle_sub_##S(size_t, size_t, const size_t*, const E*, const E*, E*);                                     \
    void oracle_mul_##S(size_t, size_t, const size_t*, const E*, const E*, E*);                                     \
    void oracle_div_##S(size_t, size_t, const size_t*, const E*, const E*, E*);                                     \
    void oracle_add_inplace_##S(size_t, size_t, const size_t*, E*, const E*);                                       \
    void oracle_sub_inplace_##S(size_t, size_t, const size_t*, E*, const E*);                                       \
    void oracle_neg_##S(size_t, size_t, const size_t*, const E*, E*);                                               \
    void oracle_sqrt_##S(size_t, size_t, const size_t*, const E*, E*);                                              \
    void oracle_square_##S(size_t, size_t, const size_t*, const E*, E*);                                            \
    void oracle_relu_##S(size_t, size_t, const size_t*, const E*, E*);                                              \
    void oracle_tanh_##S(size_t, size_t, const size_t*, const E*, E*);                                              \
    void oracle_gelu_##S(size_t, size_t, const size_t*, const E*, E*);                                              \
    void oracle_exp_##S(size_t, size_t, const size_t*, const E*, E*);                                               \
    void oracle_add_scalar_##S(size_t, size_t, const size_t*, const E*, E, E*);                                     \
    void oracle_mul_scalar_##S(size_t, size_t, const size_t*, const E*, E, E*);                                     \
    void oracle_div_scalar_##S(size_t, size_t, const size_t*, const E*, E, E*);                                     \
    void oracle_pow_##S(size_t, size_t, const size_t*, const E*, E, E*);                                            \
    void oracle_gt_scalar_##S(size_t, size_t, const size_t*, const E*, E, uint8_t*);                                \
    void oracle_sum_##S(size_t, size_t, size_t, const size_t*, const E*, E*);                                       \
    void oracle_mean_##S(size_t, size_t, size_t, const size_t*, const E*, E*);                                      \
    void oracle_sum_to_shape_##S(size_t, size_t, const size_t*, const E*, E*);                                      \
    void oracle_matmul_##S(size_t, const size_t*, const E*, const E*, E*);                                          \
    void oracle_matmul_backward_##S(size_t, size_t, const size_t*, const E*, const E*, const E*, E*, E*);
ORC_DECL(float, f32)
ORC_DECL(uint16_t, bf16)     // the oracle's bf16 is a struct of one uint16_t: the same bits at this boundary
void oracle_conv2d_im2col_f32(size_t, const size_t*, const float*, float*);
void oracle_conv2d_col2im_f32(size_t, const size_t*, const float*, float*);
}

struct OracleBackend {
    static constexpr const char* name = "oracle";
    static void* alloc(size_t bytes) { return std::malloc(bytes); }
    static void free(void* p) { std::free(p); }
    static void sync() {}
    static void discard(void*, size_t) {}
    static void h2d(void* d, const void* s, size_t n) { std::memcpy(d, s, n); }
    static void d2h(void* d, const void* s, size_t n) { std::memcpy(d, s, n); }
    static void check() {}
    static constexpr bool has_graphs = false;
    static constexpr bool has_fused_adam = false;
    static constexpr bool has_fused_nn = false;
    static constexpr bool has_cols_matmul = false;
    static constexpr bool has_conv_forward_product = false;
    static constexpr bool has_col2im_add = false;
    static constexpr auto im2col = &oracle_conv2d_im2col_f32;
    static constexpr auto col2im = &oracle_conv2d_col2im_f32;
    // with_dtype on the host, element by element, as the reference does (crates/maidenx_core/src/buffer/mod.rs:155-196)
    static void cast_bf16_f32(size_t n, const uint16_t* in, float* out) { for (size_t i = 0; i < n; ++i) out[i] = mxt::bf16_to_f32(in[i]); }
    static void cast_f32_bf16(size_t n, const float* in, uint16_t* out) { for (size_t i = 0; i < n; ++i) out[i] = mxt::f32_to_bf16(in[i]); }
    template <class E> struct K;
};
template <class E> inline E orc_one();
template <> inline float orc_one<float>() { return 1.0f; }
template <> inline uint16_t orc_one<uint16_t>() { return 0x3F80; }
#define MXT_ORC_KERNELS(E, S)                                                                                          \
    template <> struct OracleBackend::K<E> {                                                                             \
        using Bin = void (*)(size_t, size_t, const size_t*, const E*, const E*, E*);                                     \
        using Inp = void (*)(size_t, size_t, const size_t*, E*, const E*);                                               \
        using Un = void (*)(size_t, size_t, const size_t*, const E*, E*);                                                \
        using Unc = void (*)(size_t, size_t, const size_t*, const E*, E, E*);                                            \
        using Red = void (*)(size_t, size_t, size_t, const size_t*, const E*, E*);                                       \
        static constexpr Bin bin[4] = {&oracle_add_##S, &oracle_sub_##S, &oracle_mul_##S, &oracle_div_##S};              \
        static constexpr Inp inplace[2] = {&oracle_add_inplace_##S, &oracle_sub_inplace_##S};                            \
        static constexpr Un un[7] = {&oracle_neg_##S, &oracle_square_##S, &oracle_relu_##S, &oracle_tanh_##S, &oracle_gelu_##S, &oracle_exp_##S, &oracle_sqrt_##S}; \
        static constexpr Unc unc[4] = {&oracle_add_scalar_##S, &oracle_mul_scalar_##S, &oracle_div_scalar_##S, &oracle_pow_##S}; \
        static constexpr Red red[2] = {&oracle_sum_##S, &oracle_mean_##S};                                               \
        static constexpr auto gt_scalar = &oracle_gt_scalar_##S;                                                         \
        static constexpr auto sum_to_shape = &oracle_sum_to_shape_##S;                                                   \
        static constexpr auto matmul = &oracle_matmul_##S;                                                               \
        static constexpr auto matmul_backward = &oracle_matmul_backward_##S;                                             \
        /* The reference does these on the host as well. */                                                             \
        static void fill(size_t n, E* p, E v) { for (size_t i = 0; i < n; ++i) p[i] = v; }                               \
        static void cast_from_bool(size_t n, const uint8_t* in, E* out) { for (size_t i = 0; i < n; ++i) out[i] = in[i] ? orc_one<E>() : E(0); } \
        /* crates/maidenx_tensor/src/f.rs:19-24: element by element through the logical index */                        \
        static void copy_strided(size_t n, size_t nd, const size_t* md, const E* in, E* out) {                           \
            const size_t *dims = md, *strides = md + nd;                                                                 \
            const size_t off = md[2 * nd];                                                                               \
            for (size_t i = 0; i < n; ++i) {                                                                             \
                size_t rem = i, src = off;                                                                               \
                for (size_t d = nd; d-- > 0;) {                                                                          \
                    src += (rem % dims[d]) * strides[d];                                                                 \
                    rem /= dims[d];                                                                                      \
                }                                                                                                        \
                out[i] = in[src];                                                                                        \
            }                                                                                                            \
        }                                                                                                                \
        static void broadcast_scalar(size_t n, const E* src, E* dst) { fill(n, dst, *src); } /* transform.rs:328-331 */  \
    };
MXT_ORC_KERNELS(float, f32)
MXT_ORC_KERNELS(uint16_t, bf16)
using MxtBackend = OracleBackend;
#include "../maidenx_amd/host/mx_capi.hpp"
