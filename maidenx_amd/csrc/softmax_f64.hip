// Softmax along one dim for f64.  Replaces cuda_softmax_f64 of crates/maidenx_cuda/src/nn/activation/softmax.rs:26-31
// with the CPU semantics of crates/maidenx_cpu/src/nn/activation/softmax.rs:62-207: per slice m = max from -inf with
// `x > m`, s = exp(-inf - m) + sum exp(x - m), out = exp(x - m) / s, output contiguous; `dim` out of range means the
// last dim.  Everything is formed in f64 (the device library's exp, within 1 ulp of the host's); a contiguous last-dim
// row is shared by a 256-thread block (or, shorter than 128, by 8 to 64 lanes) and summed in a fixed tree order; long
// contiguous columns are split among the 16 waves of a block; every other layout is walked by one thread per slice in
// the reference's own order, strided inputs with its index rule (leading dims decomposed from dim 0 upwards).
#include <cmath>

#include "elementwise.hpp"
#include "mxh.hpp"
#include "ops.hpp"

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

// Contiguous last dim, rows shorter than 128: TPR lanes per row (8, 16, 32 or 64, at most two elements a lane), several
// rows to a wave; maxima and sums meet in a butterfly over the row's lanes.
template <int TPR>
__global__ __launch_bounds__(SFB) void softmax_shortrow_f64_kernel(const double* __restrict__ in, double* __restrict__ out, size_t rows, size_t D) {
    const size_t row = (size_t)blockIdx.x * (SFB / TPR) + threadIdx.x / TPR;
    const unsigned t = threadIdx.x % TPR;
    const bool live = row < rows;
    const double* src = in + (live ? row : 0) * D;
    double m = -INFINITY;
    if (live) for (size_t i = t; i < D; i += TPR) { double x = src[i]; m = x > m ? x : m; }
#pragma unroll
    for (int off = TPR / 2; off > 0; off >>= 1) { double o = __shfl_xor(m, off, 64); m = o > m ? o : m; }
    double s = 0.0;
    if (live) for (size_t i = t; i < D; i += TPR) s += exp(src[i] - m);
#pragma unroll
    for (int off = TPR / 2; off > 0; off >>= 1) s += __shfl_xor(s, off, 64);
    s = exp(-INFINITY - m) + s;
    if (live) for (size_t i = t; i < D; i += TPR) out[row * D + i] = exp(src[i] - m) / s;
}

// [pre, D, post] contiguous, post > 1, D >= 64: a block of 16 waves shares 64 columns (the lanes: 512 bytes of a row) and
// splits D among its waves; the waves' maxima and sums meet in LDS, the sums in wave order.  Three passes over the
// block's slab, the second and third from cache.
constexpr int SCW = 16;
__global__ __launch_bounds__(64 * SCW) void softmax_col_f64_kernel(const double* __restrict__ in, double* __restrict__ out, size_t D, size_t post,
                                                                   uint32_t jblocks) {
    const int lane = threadIdx.x % 64, w = threadIdx.x / 64;
    const uint32_t jb = blockIdx.x % jblocks;
    const size_t pre_idx = blockIdx.x / jblocks, j = (size_t)jb * 64 + lane;
    const bool live = j < post;
    const double* src = in + pre_idx * D * post + (live ? j : 0);
    double* dst = out + pre_idx * D * post + j;
    const size_t per = (D + SCW - 1) / SCW;
    const size_t l0 = (size_t)w * per < D ? (size_t)w * per : D, l1 = l0 + per < D ? l0 + per : D;
    __shared__ double red[SCW][64];
    double m = -INFINITY;
    if (live) {
#pragma unroll 4
        for (size_t l = l0; l < l1; ++l) { double x = src[l * post]; m = x > m ? x : m; }
    }
    red[w][lane] = m;
    __syncthreads();
    m = red[0][lane];
#pragma unroll
    for (int k = 1; k < SCW; ++k) m = red[k][lane] > m ? red[k][lane] : m;
    __syncthreads();
    double s = 0.0;
    if (live) {
#pragma unroll 4
        for (size_t l = l0; l < l1; ++l) s += exp(src[l * post] - m);
    }
    red[w][lane] = s;
    __syncthreads();
    s = exp(-INFINITY - m);
#pragma unroll
    for (int k = 0; k < SCW; ++k) s = s + red[k][lane];
    if (live) {
#pragma unroll 4
        for (size_t l = l0; l < l1; ++l) dst[l * post] = exp(src[l * post] - m) / s;
    }
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
    if (cont && post == 1) {
        auto rows_of = [&](auto kern, int tpr) { hipLaunchKernelGGL(kern, dim3((unsigned)cdiv(slices, (size_t)(SFB / tpr))), dim3(SFB), 0, stream(), src, out, slices, D); };
        if (D <= 16) rows_of(softmax_shortrow_f64_kernel<8>, 8);
        else if (D <= 32) rows_of(softmax_shortrow_f64_kernel<16>, 16);
        else if (D <= 64) rows_of(softmax_shortrow_f64_kernel<32>, 32);
        else rows_of(softmax_shortrow_f64_kernel<64>, 64);
        MXH_LAUNCH_CHECK("softmax_shortrow_f64");
        return;
    }
    // long columns and too few of them for a thread each to fill the chip
    if (cont && D >= 64 && slices < (1u << 22) && pre * cdiv(post, (size_t)64) < (1ull << 31)) {
        const uint32_t jblocks = (uint32_t)cdiv(post, (size_t)64);
        hipLaunchKernelGGL(softmax_col_f64_kernel, dim3((unsigned)(pre * jblocks)), dim3(64 * SCW), 0, stream(), src, out, D, post, jblocks);
        MXH_LAUNCH_CHECK("softmax_col_f64");
        return;
    }
    // a large strided input with at most one leading dim of more than one element: the contiguous softmax of its
    // logical-order copy (as for f32, softmax.hip)
    if (!cont) {
        size_t leading = 0;
        for (size_t d = 0; d < dim; ++d) leading += dims[d] > 1;
        if (leading <= 1 && num_els >= (1u << 18) && num_els < (1ull << 31) && nd <= 64 && !capture_open()) {
            double* tmp = (double*)scratch(num_els * sizeof(double), 1);
            if (!tmp) return;
            size_t cmd[2 * 64 + 1];
            for (size_t d = 0; d < nd; ++d) cmd[d] = dims[d];
            contiguous_strides(nd, dims, cmd + nd);
            cmd[2 * nd] = 0;
            const size_t* ins[1] = {strides};
            const void* inp[1] = {src};
            ew_launch<OpIdentity<double>>(num_els, nd, dims, cmd + nd, ins, tmp, inp, OpIdentity<double>{});
            softmax_f64(num_els, nd, dim, cmd, tmp, out);
            return;
        }
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
