// Softmax along one dim for f64.  Replaces cuda_softmax_f64 of crates/maidenx_cuda/src/nn/activation/softmax.rs:26-31
// with the CPU semantics of crates/maidenx_cpu/src/nn/activation/softmax.rs:62-207: per slice m = max from -inf with
// `x > m`, s = exp(-inf - m) + sum exp(x - m), out = exp(x - m) / s, output contiguous; `dim` out of range means the
// last dim.  Everything is formed in f64 (the device library's exp, within 1 ulp of the host's); a contiguous last-dim
// row is shared by a 256-thread block and summed in a fixed tree order, every other layout is walked by one thread per
// slice in the reference's own order, strided inputs with its index rule (leading dims decomposed from dim 0 upwards).
#include <cmath>

#include "mxh.hpp"

namespace mxh {

constexpr int SFB = 256;

__global__ __launch_bounds__(SFB) void softmax_row_f64_kernel(const double* __restrict__ in, double* __restrict__ out, size_t D) {
    const double* src = in + (size_t)blockIdx.x * D;
    double* dst = out + (size_t)blockIdx.x * D;
    __shared__ double red[SFB];
    const int t = threadIdx.x;
    double m = -INFINITY;
    for (size_t i = t; i < D; i += SFB) { double x = src[i]; m = x > m ? x : m; }
    red[t] = m;
    __syncthreads();
    for (int w = SFB / 2; w > 0; w >>= 1) {
        if (t < w) red[t] = red[t + w] > red[t] ? red[t + w] : red[t];
        __syncthreads();
    }
    m = red[0];
    __syncthreads();
    double s = 0.0;
    for (size_t i = t; i < D; i += SFB) s += exp(src[i] - m);
    red[t] = s;
    __syncthreads();
    for (int w = SFB / 2; w > 0; w >>= 1) {
        if (t < w) red[t] = red[t] + red[t + w];
        __syncthreads();
    }
    s = exp(-INFINITY - m) + red[0];
    for (size_t i = t; i < D; i += SFB) dst[i] = exp(src[i] - m) / s;
}

struct SoftmaxStridedF64 {
    int nd, dim, cont;
    uint32_t dims[MAXD];
    int64_t strides[MAXD];
};

__global__ __launch_bounds__(SFB) void softmax_slice_f64_kernel(SoftmaxStridedF64 sp, const double* __restrict__ in, double* __restrict__ out,
                                                                size_t slices, size_t D, size_t post) {
    size_t s_id = (size_t)blockIdx.x * SFB + threadIdx.x;
    if (s_id >= slices) return;
    size_t pre_idx = s_id / post, post_idx = s_id % post;
    int64_t base = 0, st = (int64_t)post;
    if (sp.cont) base = (int64_t)(pre_idx * D * post + post_idx);
    else {
        size_t rem = pre_idx;
        for (int d = 0; d < sp.dim; ++d) { base += (int64_t)(rem % sp.dims[d]) * sp.strides[d]; rem /= sp.dims[d]; }
        rem = post_idx;
        for (int d = sp.nd - 1; d > sp.dim; --d) { base += (int64_t)(rem % sp.dims[d]) * sp.strides[d]; rem /= sp.dims[d]; }
        st = sp.strides[sp.dim];
    }
    double* dst = out + pre_idx * D * post + post_idx;
    double m = -INFINITY;
    for (size_t i = 0; i < D; ++i) { double x = in[base + (int64_t)i * st]; m = x > m ? x : m; }
    double s = exp(-INFINITY - m);
    for (size_t i = 0; i < D; ++i) s = s + exp(in[base + (int64_t)i * st] - m);
    for (size_t i = 0; i < D; ++i) dst[i * post] = exp(in[base + (int64_t)i * st] - m) / s;
}

static void softmax_f64(size_t num_els, size_t nd, size_t dim_arg, const size_t* md, const double* in, double* out) {
    if (!md || !in || !out) return;       // the reference returns silently (softmax.rs:66-68)
    if (nd == 0 || num_els == 0) return;
    const size_t dim = dim_arg >= nd ? nd - 1 : dim_arg;
    const size_t* dims = md;
    const size_t* strides = md + nd;
    const size_t offset = md[2 * nd];
    size_t pre = 1, post = 1;
    for (size_t d = 0; d < dim; ++d) pre *= dims[d];
    for (size_t d = dim + 1; d < nd; ++d) post *= dims[d];
    const size_t D = dims[dim], slices = pre * post;
    if (D == 0 || slices == 0) return;
    bool cont = true;       // the strict test of softmax.rs:88-100
    {
        size_t acc = 1;
        for (size_t d = nd; d-- > 0;) {
            if (strides[d] != acc) { cont = false; break; }
            acc *= dims[d];
        }
    }
    const double* src = in + offset;
    if (slices >= (1ull << 31)) { set_status(ERR_TOO_LARGE, "softmax: 2^31 or more slices"); return; }
    if (cont && post == 1 && D >= 128) {
        hipLaunchKernelGGL(softmax_row_f64_kernel, dim3((unsigned)slices), dim3(SFB), 0, stream(), src, out, D);
        MXH_LAUNCH_CHECK("softmax_row_f64");
        return;
    }
    if (!cont && nd > (size_t)MAXD) { set_status(ERR_UNSUPPORTED, "softmax: strided input of rank above 8"); return; }
    SoftmaxStridedF64 sp;
    sp.nd = (int)nd; sp.dim = (int)dim; sp.cont = cont ? 1 : 0;
    for (int d = 0; d < MAXD; ++d) {
        sp.dims[d] = d < (int)nd && !cont ? (uint32_t)dims[d] : 1;
        sp.strides[d] = d < (int)nd && !cont ? (int64_t)strides[d] : 0;
    }
    hipLaunchKernelGGL(softmax_slice_f64_kernel, dim3(cdiv(slices, SFB)), dim3(SFB), 0, stream(), sp, src, out, slices, D, post);
    MXH_LAUNCH_CHECK("softmax_slice_f64");
}

}  // namespace mxh

extern "C" void hip_softmax_f64(size_t num_els, size_t num_dims, size_t dim, const size_t* md, const double* in, double* out) { MXH_API;
    mxh::softmax_f64(num_els, num_dims, dim, md, in, out);
}
