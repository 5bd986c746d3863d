// TEST INFRASTRUCTURE ONLY — CPU restatement of crates/maidenx_cpu/src/nn/activation/softmax.rs.
// Metadata (softmax.rs:76-78): dims[n] | strides[n] | offset; `dim` is a separate argument and an
// out-of-range value means the last dim (:74).  All arithmetic is in the storage dtype: for bf16 every
// subtraction, exp, add and division rounds (softmax.rs:46-53 and the `half` operators).
// Kept as the source has them:
//   * the contiguity test is the strict one (:88-100): a size-1 dim with an odd stride makes the
//     input "non-contiguous";
//   * the non-contiguous index (:120-136) decomposes pre_idx from dim 0 upwards (dim 0 fastest),
//     post_idx from the last dim downwards;
//   * the running sum starts from exp(-inf - max) (:143): 0 for a finite or +inf maximum, NaN when the
//     maximum is still -inf (an all -inf or all-NaN slice).
#include "common.hpp"

using namespace orc;

namespace {

template <typename T> struct F;
template <> struct F<float> {
    static float neg_inf() { return -std::numeric_limits<float>::infinity(); }
    static float exp(float x) { return std::exp(x); }
};
template <> struct F<double> {
    static double neg_inf() { return -std::numeric_limits<double>::infinity(); }
    static double exp(double x) { return std::exp(x); }
};
template <class C> struct F<half_t<C>> {
    static half_t<C> neg_inf() { return half_t<C>::from_f32(-std::numeric_limits<float>::infinity()); }
    static half_t<C> exp(half_t<C> x) { return half_t<C>::from_f32(std::exp(x.to_f32())); }
};

template <typename T>
void softmax(size_t num_els, size_t nd, size_t dim_arg, const size_t* md, const T* in, T* out) {
    (void)num_els;
    if (!md || !in || !out) return;
    const size_t dim = dim_arg >= nd ? nd - 1 : dim_arg;
    const size_t* dims = md;
    const size_t* strides = md + nd;
    const size_t offset = md[2 * nd];
    size_t pre = 1, post = 1;
    for (size_t d = 0; d < dim; ++d) pre *= dims[d];
    for (size_t d = dim + 1; d < nd; ++d) post *= dims[d];
    const size_t D = dims[dim];
    bool cont = true;
    {
        size_t acc = 1;
        for (size_t d = nd; d-- > 0;) {
            if (strides[d] != acc) { cont = false; break; }
            acc *= dims[d];
        }
    }
    auto index = [&](size_t pre_idx, size_t i, size_t post_idx) {
        if (cont) return offset + pre_idx * (D * post) + i * post + post_idx;
        size_t idx = offset, rem = pre_idx;
        for (size_t d = 0; d < dim; ++d) { idx += (rem % dims[d]) * strides[d]; rem /= dims[d]; }
        idx += i * strides[dim];
        rem = post_idx;
        for (size_t d = nd; d-- > dim + 1;) { idx += (rem % dims[d]) * strides[d]; rem /= dims[d]; }
        return idx;
    };
    const size_t slices = pre * post;
    ORC_PAR_FOR
    for (size_t s = 0; s < slices; ++s) {
        const size_t pre_idx = s / post, post_idx = s % post;
        T mx = F<T>::neg_inf();
        for (size_t i = 0; i < D; ++i) {
            T v = in[index(pre_idx, i, post_idx)];
            if (v > mx) mx = v;
        }
        T sum = F<T>::exp(F<T>::neg_inf() - mx);
        for (size_t i = 0; i < D; ++i) sum = sum + F<T>::exp(in[index(pre_idx, i, post_idx)] - mx);
        for (size_t i = 0; i < D; ++i)
            out[pre_idx * (D * post) + i * post + post_idx] = F<T>::exp(in[index(pre_idx, i, post_idx)] - mx) / sum;
    }
}

}  // namespace

#define ORC_SOFTMAX_FOR(T, SUF)                                                                                       \
    extern "C" void oracle_softmax_##SUF(size_t n, size_t nd, size_t dim, const size_t* md, const T* in, T* out) {    \
        softmax<T>(n, nd, dim, md, in, out);                                                                          \
    }

ORC_SOFTMAX_FOR(float, f32)
ORC_SOFTMAX_FOR(double, f64)
ORC_SOFTMAX_FOR(bf16, bf16)
ORC_SOFTMAX_FOR(f16, f16)
