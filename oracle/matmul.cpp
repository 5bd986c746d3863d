// TEST INFRASTRUCTURE ONLY — CPU restatement of crates/maidenx_cpu/src/ops/matmul.rs.
// Metadata layout (matmul.rs:24-40):
//   out_ndim, a_ndim, b_ndim | out_shape | a_shape | b_shape | a_strides | b_strides | a_off | b_off
// The accumulator has the storage dtype and k runs ascending, multiply and add unfused
// (build with -ffp-contract=off); each output element is produced by one task, so the
// result is deterministic whatever the thread count.
#include <algorithm>

#include "common.hpp"

using namespace orc;

namespace {

// `acc += a * b`.  For the integer dtypes an overflow wraps (the reference's release build; a panic in its debug build):
// done in the unsigned type, where C++ defines it.
template <typename T> inline T mac(T acc, T a, T b) {
    if constexpr (std::is_integral<T>::value) {
        using U = typename std::make_unsigned<T>::type;
        return (T)(U)((U)acc + (U)((U)a * (U)b));
    } else {
        acc += a * b;
        return acc;
    }
}


template <typename T> inline T zero_of() { return T(0); }
template <> inline bf16 zero_of<bf16>() { return bf16::from_f32(0.0f); }
template <> inline f16 zero_of<f16>() { return f16::from_f32(0.0f); }

struct MM {
    size_t out_ndim, a_ndim, b_ndim;
    const size_t *out_shape, *a_shape, *b_shape, *a_strides, *b_strides;
    size_t a_off, b_off;
};
inline MM parse(const size_t* md) {
    MM p;
    p.out_ndim = md[0]; p.a_ndim = md[1]; p.b_ndim = md[2];
    p.out_shape = md + 3;
    p.a_shape = p.out_shape + p.out_ndim;
    p.b_shape = p.a_shape + p.a_ndim;
    p.a_strides = p.b_shape + p.b_ndim;
    p.b_strides = p.a_strides + p.a_ndim;
    p.a_off = p.b_strides[p.b_ndim];
    p.b_off = p.b_strides[p.b_ndim + 1];
    return p;
}

// matmul_op! (matmul.rs:5-122)
template <typename T>
void matmul(size_t num_els, const size_t* md, const T* a, const T* b, T* c) {
    if (!md || !a || !b || !c) return;
    MM p = parse(md);
    if (p.a_ndim == 0 || p.b_ndim == 0) return;
    size_t m = p.out_ndim >= 2 ? p.out_shape[p.out_ndim - 2] : 1;
    size_t n = p.out_ndim >= 1 ? p.out_shape[p.out_ndim - 1] : 1;
    size_t k = p.a_ndim >= 1 ? p.a_shape[p.a_ndim - 1] : 1;
    if (m == 0 || n == 0 || k == 0) return;
    bool a_cont = is_contiguous(p.a_ndim, p.a_shape, p.a_strides);
    bool b_cont = is_contiguous(p.b_ndim, p.b_shape, p.b_strides);
    size_t a_size = num_els * k, b_size = num_els * k;   // :53-54, the guards below use these
    const T* as = a + p.a_off;
    const T* bs = b + p.b_off;
    size_t rows = (num_els + n - 1) / n;                  // par_chunks_mut(n)
    ORC_PAR_FOR
    for (size_t batch_m = 0; batch_m < rows; ++batch_m) {
        size_t batch_idx = batch_m / m, m_idx = batch_m % m;
        size_t row_len = std::min(n, num_els - batch_m * n);
        T* c_row = c + batch_m * n;
        for (size_t n_idx = 0; n_idx < n; ++n_idx) {
            T acc = zero_of<T>();
            if (a_cont && b_cont) {
                size_t a_base = batch_idx * (m * k) + m_idx * k;
                size_t b_base = batch_idx * (k * n);
                for (size_t k_idx = 0; k_idx < k; ++k_idx) {
                    size_t ai = a_base + k_idx, bi = b_base + k_idx * n + n_idx;
                    if (ai < a_size && bi < b_size) acc = mac(acc, as[ai], bs[bi]);
                }
            } else {
                // :87-113 — the batch stride is strides[0] whatever the rank
                for (size_t k_idx = 0; k_idx < k; ++k_idx) {
                    size_t ai = p.a_ndim >= 2 ? batch_idx * p.a_strides[0] + m_idx * p.a_strides[p.a_ndim - 2] +
                                                    k_idx * p.a_strides[p.a_ndim - 1]
                                              : k_idx * p.a_strides[0];
                    size_t bi = p.b_ndim >= 2 ? batch_idx * p.b_strides[0] + k_idx * p.b_strides[p.b_ndim - 2] +
                                                    n_idx * p.b_strides[p.b_ndim - 1]
                                              : n_idx * p.b_strides[0];
                    if (ai < a_size && bi < b_size) acc = mac(acc, as[ai], bs[bi]);
                }
            }
            if (n_idx < row_len) c_row[n_idx] = acc;
        }
    }
}

// matmul_backward_op! (matmul.rs:124-268): contiguous indexing only, strides ignored.
template <typename T>
void matmul_backward(size_t num_els_a, size_t num_els_b, const size_t* md, const T* grad_output, const T* a,
                     const T* b, T* grad_a, T* grad_b) {
    if (!md || !grad_output || !a || !b) return;
    MM p = parse(md);
    if (p.a_ndim == 0 || p.b_ndim == 0) return;
    size_t m = p.out_ndim >= 2 ? p.out_shape[p.out_ndim - 2] : 1;
    size_t n = p.out_ndim >= 1 ? p.out_shape[p.out_ndim - 1] : 1;
    size_t k = p.b_ndim >= 2 ? p.b_shape[p.b_ndim - 2] : (p.a_ndim >= 1 ? p.a_shape[p.a_ndim - 1] : 1);
    if (m == 0 || n == 0 || k == 0) return;
    size_t go_size = 1;
    for (size_t d = 0; d < p.out_ndim; ++d) go_size *= p.out_shape[d];
    if (go_size == 0) return;
    const T* go = grad_output;
    if (grad_a) {
        const T* bs = b + p.b_off;
        size_t rows = (num_els_a + k - 1) / k;
        ORC_PAR_FOR
        for (size_t batch_m = 0; batch_m < rows; ++batch_m) {
            size_t batch_idx = batch_m / m, m_idx = batch_m % m;
            size_t row_len = std::min(k, num_els_a - batch_m * k);
            T* g_row = grad_a + batch_m * k;
            for (size_t k_idx = 0; k_idx < k; ++k_idx) {
                T acc = zero_of<T>();
                if (p.out_ndim == 0) {
                    if (k_idx < num_els_b) acc = go[0] * bs[k_idx];
                } else {
                    size_t g_base = batch_idx * (m * n) + m_idx * n, b_base = batch_idx * (k * n);
                    for (size_t n_idx = 0; n_idx < n; ++n_idx)
                        if (g_base + n_idx < go_size && b_base + k_idx * n + n_idx < num_els_b)
                            acc = mac(acc, go[g_base + n_idx], bs[b_base + k_idx * n + n_idx]);
                }
                if (k_idx < row_len) g_row[k_idx] = acc;
            }
        }
    }
    if (grad_b) {
        const T* as = a + p.a_off;
        size_t rows = (num_els_b + n - 1) / n;
        ORC_PAR_FOR
        for (size_t batch_k = 0; batch_k < rows; ++batch_k) {
            size_t batch_idx = batch_k / k, k_idx = batch_k % k;
            size_t row_len = std::min(n, num_els_b - batch_k * n);
            T* g_row = grad_b + batch_k * n;
            for (size_t n_idx = 0; n_idx < n; ++n_idx) {
                T acc = zero_of<T>();
                if (p.out_ndim == 0) {
                    if (k_idx < num_els_a) acc = go[0] * as[k_idx];
                } else {
                    size_t a_base = batch_idx * (m * k), g_base = batch_idx * (m * n);
                    for (size_t m_idx = 0; m_idx < m; ++m_idx) {
                        size_t ai = a_base + m_idx * k + k_idx, gi = g_base + m_idx * n + n_idx;
                        if (ai < num_els_a && gi < go_size) acc = mac(acc, as[ai], go[gi]);
                    }
                }
                if (n_idx < row_len) g_row[n_idx] = acc;
            }
        }
    }
}

}  // namespace

#define ORC_MATMUL_FOR(T, SUF)                                                                              \
    extern "C" void oracle_matmul_##SUF(size_t num_els, const size_t* md, const T* a, const T* b, T* c) {   \
        matmul<T>(num_els, md, a, b, c);                                                                    \
    }                                                                                                       \
    extern "C" void oracle_matmul_backward_##SUF(size_t na, size_t nb, const size_t* md, const T* go,       \
                                                 const T* a, const T* b, T* ga, T* gb) {                    \
        matmul_backward<T>(na, nb, md, go, a, b, ga, gb);                                                   \
    }

ORC_MATMUL_FOR(float, f32)
ORC_MATMUL_FOR(double, f64)
ORC_MATMUL_FOR(bf16, bf16)
ORC_MATMUL_FOR(f16, f16)
ORC_MATMUL_FOR(uint8_t, u8)
ORC_MATMUL_FOR(uint16_t, u16)
ORC_MATMUL_FOR(uint32_t, u32)
ORC_MATMUL_FOR(uint64_t, u64)
ORC_MATMUL_FOR(int8_t, i8)
ORC_MATMUL_FOR(int16_t, i16)
ORC_MATMUL_FOR(int32_t, i32)
ORC_MATMUL_FOR(int64_t, i64)
