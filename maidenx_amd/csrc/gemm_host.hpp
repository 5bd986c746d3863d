// Host side of matmul / matmul_backward: the reference's metadata (crates/maidenx_cpu/src/ops/matmul.rs:24-40, 147-160)
// turned into strided batched products `out[b,i,j] = sum_r X[b,i,r] * Y[b,r,j]`, handed to the dispatch of the dtype.
#pragma once
#include "gemm_small.hpp"
#include "mxh.hpp"

namespace mxh {

struct MMeta {
    size_t out_ndim, a_ndim, b_ndim;
    const size_t *out_shape, *a_shape, *b_shape, *a_strides, *b_strides;
    size_t a_off, b_off;
};
static inline MMeta parse_mm(const size_t* md) {
    MMeta p;
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

// matmul.rs:5-122
template <class T, class Dispatch>
void matmul_fwd(size_t num_els, const size_t* md, const T* a, const T* b, T* c, Dispatch gemm_dispatch_fn) {
    if (!md || !a || !b || !c) return;                    // the reference returns silently
    MMeta p = parse_mm(md);
    if (p.a_ndim == 0 || p.b_ndim == 0) return;
    size_t m = p.out_ndim >= 2 ? p.out_shape[p.out_ndim - 2] : 1;
    size_t n = p.out_ndim >= 1 ? p.out_shape[p.out_ndim - 1] : 1;
    size_t k = p.a_shape[p.a_ndim - 1];
    if (m == 0 || n == 0 || k == 0 || num_els == 0) return;
    if (num_els % (m * n) != 0 || m >= (1ull << 31) || n >= (1ull << 31) || k >= (1ull << 31)) {
        set_status(ERR_INVALID, "matmul: num_els is not batch*m*n or an extent is 2^31 or more");
        return;
    }
    // (the reference indexes b with a's reduction length whatever b's shape says; a caller whose shapes disagree would have
    // the kernels read past b)
    if (p.b_ndim >= 2 && p.b_shape[p.b_ndim - 2] != k) { set_status(ERR_INVALID, "matmul: a's last extent is not b's second to last"); return; }
    GemmArgs g{};
    g.X = a + p.a_off; g.Y = b + p.b_off; g.out = c;
    g.I = (uint32_t)m; g.J = (uint32_t)n; g.R = (uint32_t)k; g.batch = (uint32_t)(num_els / (m * n));
    bool a_cont = ref_is_contiguous(p.a_ndim, p.a_shape, p.a_strides);
    bool b_cont = ref_is_contiguous(p.b_ndim, p.b_shape, p.b_strides);
    if (a_cont && b_cont) {                               // :75-86
        g.xb = (int64_t)(m * k); g.xi = (int64_t)k; g.xr = 1;
        g.yb = (int64_t)(k * n); g.yr = (int64_t)n; g.yj = 1;
    } else {                                              // :87-113, batch stride = strides[0]
        if (p.a_ndim >= 2) { g.xb = (int64_t)p.a_strides[0]; g.xi = (int64_t)p.a_strides[p.a_ndim - 2]; g.xr = (int64_t)p.a_strides[p.a_ndim - 1]; }
        else { g.xb = 0; g.xi = 0; g.xr = (int64_t)p.a_strides[0]; }
        if (p.b_ndim >= 2) { g.yb = (int64_t)p.b_strides[0]; g.yr = (int64_t)p.b_strides[p.b_ndim - 2]; g.yj = (int64_t)p.b_strides[p.b_ndim - 1]; }
        else { g.yb = 0; g.yr = 0; g.yj = (int64_t)p.b_strides[0]; }
    }
    gemm_dispatch_fn(g);
}

// matmul.rs:124-268 — contiguous indexing, strides ignored, either gradient may be null.
template <class T, class Dispatch>
void matmul_bwd(size_t num_els_a, size_t num_els_b, const size_t* md, const T* go, const T* a, const T* b, T* ga, T* gb, Dispatch gemm_dispatch_fn) {
    if (!md || !go || !a || !b) return;
    MMeta p = parse_mm(md);
    if (p.a_ndim == 0 || p.b_ndim == 0) return;
    size_t m = p.out_ndim >= 2 ? p.out_shape[p.out_ndim - 2] : 1;
    size_t n = p.out_ndim >= 1 ? p.out_shape[p.out_ndim - 1] : 1;
    size_t k = p.b_ndim >= 2 ? p.b_shape[p.b_ndim - 2] : p.a_shape[p.a_ndim - 1];
    if (m == 0 || n == 0 || k == 0) return;
    if (p.out_ndim == 0) { set_status(ERR_UNSUPPORTED, "matmul_backward: 0-d output"); return; }
    if (m >= (1ull << 31) || n >= (1ull << 31) || k >= (1ull << 31)) { set_status(ERR_INVALID, "matmul_backward: extent of 2^31 or more"); return; }
    if (ga) {
        if (num_els_a % (m * k) != 0) { set_status(ERR_INVALID, "matmul_backward: num_els_a is not batch*m*k"); return; }
        GemmArgs g{};
        g.X = go; g.Y = b + p.b_off; g.out = ga;
        g.I = (uint32_t)m; g.J = (uint32_t)k; g.R = (uint32_t)n; g.batch = (uint32_t)(num_els_a / (m * k));
        g.xb = (int64_t)(m * n); g.xi = (int64_t)n; g.xr = 1;
        g.yb = (int64_t)(k * n); g.yr = 1; g.yj = (int64_t)n;
        gemm_dispatch_fn(g);
    }
    if (gb) {
        if (num_els_b % (k * n) != 0) { set_status(ERR_INVALID, "matmul_backward: num_els_b is not batch*k*n"); return; }
        GemmArgs g{};
        g.X = a + p.a_off; g.Y = go; g.out = gb;
        g.I = (uint32_t)k; g.J = (uint32_t)n; g.R = (uint32_t)m; g.batch = (uint32_t)(num_els_b / (k * n));
        g.xb = (int64_t)(m * k); g.xi = 1; g.xr = (int64_t)k;
        g.yb = (int64_t)(m * n); g.yr = (int64_t)n; g.yj = 1;
        gemm_dispatch_fn(g);
    }
}

}  // namespace mxh
