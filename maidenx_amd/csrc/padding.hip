// Padding, forward and backward.  Replaces cuda_pad_with_{constant,reflection,replication}_<T> and their
// _backward_ partners of crates/maidenx_cuda/src/ops/padding.rs:13-71 with the CPU semantics of
// crates/maidenx_cpu/src/ops/padding.rs (constant :7-113 and :327-436; the two edge modes further down).
// Metadata: in_dims[n] | in_strides[n] | in_offset | out_dims[n] | (pad_before, pad_after)[n]
// Pure data movement, bit-exact.  One lane per 16 bytes of output; the coordinate walk uses
// multiply-high division on the collapsed shape (dims without padding whose input strides chain
// are merged, so [B,C,H,W] padded on H,W walks two divisions, not four).
#include "elementwise.hpp"
#include "ops.hpp"

namespace mxh {

struct PadSpace {
    int ndims;
    uint32_t out_dims[MAXD];
    uint32_t in_dims[MAXD];
    uint32_t before[MAXD];
    FastDiv div[MAXD];
    int64_t in_strides[MAXD];
    // the innermost dim, kept apart: a thread's elements mostly differ in this coordinate only
    uint32_t out_last, in_last, before_last;
    int64_t stride_last;
    FastDiv div_last;
};


constexpr int PB = 256;

// The type the backward sums are formed in and its conversions: f32 for the three float formats of 32 or 16 bits (one
// rounding at the end for the 16-bit ones), the storage type itself for f64.
template <class T> struct PadAcc {
    using A = float;
    static __device__ A ld(T v) { return Ar<T>::to_f32(v); }
    static __device__ T st(A a) { return Ar<T>::from_f32(a); }
};
template <> struct PadAcc<double> {
    using A = double;
    static __device__ A ld(double v) { return v; }
    static __device__ double st(A a) { return a; }
};
// The integers sum in the storage type and wrap (the reference's release build; its debug build panics on overflow):
// formed in the unsigned type, where wrapping is defined, which also makes the sums independent of their order.
template <class T> struct PadAccInt {
    using A = typename std::make_unsigned<T>::type;
    static __device__ A ld(T v) { return (A)v; }
    static __device__ T st(A a) { return (T)a; }
};
template <> struct PadAcc<uint8_t> : PadAccInt<uint8_t> {};
template <> struct PadAcc<uint16_t> : PadAccInt<uint16_t> {};
template <> struct PadAcc<uint32_t> : PadAccInt<uint32_t> {};
template <> struct PadAcc<uint64_t> : PadAccInt<uint64_t> {};
template <> struct PadAcc<int8_t> : PadAccInt<int8_t> {};
template <> struct PadAcc<int16_t> : PadAccInt<int16_t> {};
template <> struct PadAcc<int32_t> : PadAccInt<int32_t> {};
template <> struct PadAcc<int64_t> : PadAccInt<int64_t> {};
enum EdgeMode : int { EDGE_REFLECT = 0, EDGE_REPLICATE = 1, EDGE_NONE = 2 };     // NONE: constant padding, whose border feeds nothing back

// forward: out[i] = inside ? in[idx] : pad_value
// backward (FWD = false): grad_in[idx] = 0 + grad_out[i] for every inside i
// A thread owns Q consecutive output elements: one coordinate decomposition (multiply-high divisions); the outer
// coordinates ("the row") are located once and again only when the elements run past the end of a row, so an
// element costs one compare and one add.  The contiguous side (out for forward, grad_out for backward) moves
// as one Q-element vector.
template <class T, bool FWD, int Q>
__global__ __launch_bounds__(PB) void pad_const_kernel(PadSpace sp, const T* __restrict__ src, T* __restrict__ dst,
                                                       size_t n_out, T pad_value) {
    size_t i0 = ((size_t)blockIdx.x * PB + threadIdx.x) * Q;
    if (i0 >= n_out) return;
    // coordinates: x in the innermost dim, c[d] in the outer ones
    uint32_t c[MAXD];
    uint32_t x;
    {
        uint32_t r = (uint32_t)i0;
        if (sp.ndims > 1) fd_divmod(r, sp.div_last, r, x);
        else { x = r; r = 0; }
#pragma unroll
        for (int d = MAXD - 2; d >= 0; --d) {
            if (d >= sp.ndims - 1) { c[d] = 0; continue; }
            uint32_t q, m;
            if (d > 0) fd_divmod(r, sp.div[d], q, m);
            else { q = 0; m = r; }
            c[d] = m;
            r = q;
        }
    }
    // the row (all outer coordinates): inside the input or not, and where it starts
    bool row_in;
    int64_t row_idx;
    auto locate_row = [&]() {
        row_in = true;
        row_idx = 0;
#pragma unroll
        for (int d = 0; d < MAXD - 1; ++d) {
            if (d >= sp.ndims - 1) break;
            uint32_t ic = c[d] - sp.before[d];           // wraps when c < before → fails the test below
            row_in = row_in && ic < sp.in_dims[d];
            row_idx += (int64_t)ic * sp.in_strides[d];
        }
    };
    locate_row();
    const bool full = i0 + Q <= n_out;
    AVec<T, Q> v;
    if constexpr (!FWD) {
        if (full) v = *(const AVec<T, Q>*)(src + i0);
        else
            for (int e = 0; e < Q; ++e) v.v[e] = i0 + e < n_out ? src[i0 + e] : T{};
    }
#pragma unroll
    for (int e = 0; e < Q; ++e) {
        const uint32_t ic = x - sp.before_last;
        const bool inside = row_in && ic < sp.in_last && (full || i0 + e < n_out);
        const int64_t idx = row_idx + (int64_t)ic * sp.stride_last;
        if constexpr (FWD) {
            v.v[e] = inside ? src[idx] : pad_value;
        } else {
            if (inside) {
                T g = v.v[e];
                dst[idx] = PadAcc<T>::st((typename PadAcc<T>::A)0 + PadAcc<T>::ld(g));      // −0 → +0 like the reference's sums from zero
            }
        }
        // next output element; at the end of a row, carry into the outer coordinates
        if (++x == sp.out_last && e + 1 < Q) {
            x = 0;
            bool carry = true;
#pragma unroll
            for (int d = MAXD - 2; d >= 0; --d) {
                if (d >= sp.ndims - 1) continue;
                if (carry) {
                    c[d] += 1;
                    carry = c[d] == sp.out_dims[d];
                    if (carry) c[d] = 0;
                }
            }
            locate_row();
        }
    }
    if constexpr (FWD) {
        if (full) *(AVec<T, Q>*)(dst + i0) = v;
        else
            for (int e = 0; e < Q; ++e)
                if (i0 + e < n_out) dst[i0 + e] = v.v[e];
    }
}

// ---- at most three dims after merging (the usual [N*C, H, W] of a padded image batch) -------------------
// The same walks with 32-bit coordinates and two divisions per thread.  Dims are right-aligned: slot 2 is the
// innermost one, missing outer dims have size 1.
struct Pad3 {
    uint32_t out[3], in[3], before[3];
    FastDiv out_div[3], in_div[3];
    int64_t in_stride[3];
    uint32_t out_stride[3];
};
static bool make_pad3(const PadSpace& sp, Pad3& p3) {
    if (sp.ndims > 3) return false;
    const int shift = 3 - sp.ndims;
    uint64_t ost = 1;
    for (int k = 2; k >= 0; --k) {
        const int d = k - shift;
        const bool real = d >= 0;
        p3.out[k] = real ? sp.out_dims[d] : 1;
        p3.in[k] = real ? sp.in_dims[d] : 1;
        p3.before[k] = real ? sp.before[d] : 0;
        p3.in_stride[k] = real ? sp.in_strides[d] : 0;
        p3.out_div[k] = make_fastdiv(p3.out[k]);
        p3.in_div[k] = make_fastdiv(p3.in[k]);
        p3.out_stride[k] = (uint32_t)ost;
        ost *= p3.out[k];
    }
    return ost < (1ull << 31);
}

// A thread owns U vectors of Q consecutive output elements, PB*Q apart, and issues the loads of all of them before the
// first store: one vector per thread leaves too few bytes in flight per CU to cover the memory latency.  Forward loads
// are unconditional (position 0 stands in for an element outside the input), so none of them waits on a branch.
template <class T, bool FWD, int Q, int U>
__global__ __launch_bounds__(PB) void pad_const3_kernel(Pad3 sp, const T* __restrict__ src, T* __restrict__ dst, uint32_t n_out, T pad_value) {
    const uint32_t base = (blockIdx.x * (uint32_t)(U * PB) + threadIdx.x) * Q;
    AVec<T, Q> v[U];
    if constexpr (FWD) {
        bool in_mask[U][Q];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t i0 = base + (uint32_t)u * (PB * Q);
            const bool live = i0 < n_out;
            uint32_t q, c2, c1, c0;
            fd_divmod(live ? i0 : 0u, sp.out_div[2], q, c2);
            fd_divmod(q, sp.out_div[1], c0, c1);
            int64_t row = 0;
            bool row_in = false, fresh = true;
#pragma unroll
            for (int e = 0; e < Q; ++e) {
                if (fresh) {
                    const uint32_t i0c = c0 - sp.before[0], i1c = c1 - sp.before[1];      // wrap when outside: fail the test
                    row_in = i0c < sp.in[0] && i1c < sp.in[1];
                    row = (int64_t)i0c * sp.in_stride[0] + (int64_t)i1c * sp.in_stride[1];
                    fresh = false;
                }
                const uint32_t ic = c2 - sp.before[2];
                const bool inside = live && row_in && ic < sp.in[2] && i0 + e < n_out;
                const int64_t idx = row + (int64_t)ic * sp.in_stride[2];
                in_mask[u][e] = inside;
                v[u].v[e] = src[inside ? idx : 0];
                if (++c2 == sp.out[2]) {
                    c2 = 0;
                    fresh = true;
                    if (++c1 == sp.out[1]) { c1 = 0; ++c0; }
                }
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t i0 = base + (uint32_t)u * (PB * Q);
            if (i0 >= n_out) continue;
#pragma unroll
            for (int e = 0; e < Q; ++e)
                if (!in_mask[u][e]) v[u].v[e] = pad_value;
            if (i0 + Q <= n_out) *(AVec<T, Q>*)(dst + i0) = v[u];
            else
                for (int e = 0; e < Q; ++e)
                    if (i0 + e < n_out) dst[i0 + e] = v[u].v[e];
        }
    } else {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t i0 = base + (uint32_t)u * (PB * Q);
            if (i0 + Q <= n_out) v[u] = *(const AVec<T, Q>*)(src + i0);
            else
                for (int e = 0; e < Q; ++e) v[u].v[e] = i0 + e < n_out ? src[i0 + e] : T{};
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t i0 = base + (uint32_t)u * (PB * Q);
            if (i0 >= n_out) continue;
            uint32_t q, c2, c1, c0;
            fd_divmod(i0, sp.out_div[2], q, c2);
            fd_divmod(q, sp.out_div[1], c0, c1);
            int64_t row = 0;
            bool row_in = false, fresh = true;
#pragma unroll
            for (int e = 0; e < Q; ++e) {
                if (fresh) {
                    const uint32_t i0c = c0 - sp.before[0], i1c = c1 - sp.before[1];
                    row_in = i0c < sp.in[0] && i1c < sp.in[1];
                    row = (int64_t)i0c * sp.in_stride[0] + (int64_t)i1c * sp.in_stride[1];
                    fresh = false;
                }
                const uint32_t ic = c2 - sp.before[2];
                const bool inside = row_in && ic < sp.in[2] && i0 + e < n_out;
                const int64_t idx = row + (int64_t)ic * sp.in_stride[2];
                if (inside) dst[idx] = PadAcc<T>::st((typename PadAcc<T>::A)0 + PadAcc<T>::ld(v[u].v[e]));      // -0 -> +0 like the reference's sums from zero
                if (++c2 == sp.out[2]) {
                    c2 = 0;
                    fresh = true;
                    if (++c1 == sp.out[1]) { c1 = 0; ++c0; }
                }
            }
        }
    }
}

template <class T>
__global__ __launch_bounds__(PB) void zero_kernel(T* p, size_t n) {
    size_t i = (size_t)blockIdx.x * PB + threadIdx.x;
    if (i < n) p[i] = T{};
}

// Four vectors per thread once that still leaves every CU several blocks; one otherwise.
template <class T, bool FWD>
static void pad_const3_launch(const Pad3& p3, const T* src, T* dst, size_t n_out, T pad_value) {
    constexpr int Q = 16 / sizeof(T);
    const size_t vecs = cdiv(n_out, (size_t)Q);
    if (vecs >= (size_t)PB * 4 * 1024)
        hipLaunchKernelGGL((pad_const3_kernel<T, FWD, Q, 4>), dim3(cdiv(vecs, (size_t)PB * 4)), dim3(PB), 0, stream(), p3, src, dst, (uint32_t)n_out, pad_value);
    else
        hipLaunchKernelGGL((pad_const3_kernel<T, FWD, Q, 1>), dim3(cdiv(vecs, (size_t)PB)), dim3(PB), 0, stream(), p3, src, dst, (uint32_t)n_out, pad_value);
}

static bool build_space(size_t nd, const size_t* md, PadSpace& sp, size_t* in_off, bool* cont, bool* exact) {
    const size_t* in_dims = md;
    const size_t* in_strides = md + nd;
    *in_off = md[2 * nd];
    const size_t* out_dims = md + 2 * nd + 1;
    const size_t* pads = md + 3 * nd + 1;
    *cont = ref_is_contiguous(nd, in_dims, in_strides);
    size_t cs[64];
    if (nd > 64) return false;
    contiguous_strides(nd, in_dims, cs);
    const size_t* st = *cont ? cs : in_strides;     // padding.rs:76-93: contiguous inputs are indexed row-major
    *exact = true;
    int n = 0;
    uint64_t od[64], id[64], bf[64];
    int64_t is[64];
    for (size_t d = 0; d < nd; ++d) {
        if (out_dims[d] != in_dims[d] + pads[2 * d] + pads[2 * d + 1]) *exact = false;
        bool plain = pads[2 * d] == 0 && out_dims[d] == in_dims[d];
        if (plain && in_dims[d] == 1) continue;
        // merge a pad-free dim into its (pad-free) outer neighbour when the input strides chain
        if (n > 0 && plain && bf[n - 1] == 0 && od[n - 1] == id[n - 1] && (uint64_t)is[n - 1] == st[d] * in_dims[d]) {
            od[n - 1] *= out_dims[d]; id[n - 1] *= in_dims[d]; is[n - 1] = (int64_t)st[d];
        } else {
            od[n] = out_dims[d]; id[n] = in_dims[d]; bf[n] = pads[2 * d]; is[n] = (int64_t)st[d]; ++n;
        }
    }
    if (n == 0) { od[0] = id[0] = 1; bf[0] = 0; is[0] = 1; n = 1; }
    if (n > MAXD) return false;
    sp.ndims = n;
    sp.out_last = (uint32_t)od[n - 1]; sp.in_last = (uint32_t)id[n - 1]; sp.before_last = (uint32_t)bf[n - 1];
    sp.stride_last = is[n - 1];
    sp.div_last = make_fastdiv(sp.out_last);
    for (int d = 0; d < MAXD; ++d) {
        sp.out_dims[d] = d < n ? (uint32_t)od[d] : 1;
        sp.in_dims[d] = d < n ? (uint32_t)id[d] : 1;
        sp.before[d] = d < n ? (uint32_t)bf[d] : 0;
        sp.in_strides[d] = d < n ? is[d] : 0;
        sp.div[d] = make_fastdiv(sp.out_dims[d]);
    }
    return true;
}

template <class T>
void pad_forward(size_t n_in, size_t n_out, size_t nd, const size_t* md, const T* in, T* out, T pad_value) {
    (void)n_in;
    if (!md || !in || !out) { set_status(ERR_INVALID, "pad: null argument"); return; }
    if (n_out == 0) return;
    if (n_out >= (1ull << 31)) { set_status(ERR_TOO_LARGE, "pad: output of 2^31 or more elements"); return; }
    PadSpace sp; size_t off; bool cont, exact;
    if (!build_space(nd, md, sp, &off, &cont, &exact)) { set_status(ERR_UNSUPPORTED, "pad: rank above 8 after collapse"); return; }
    constexpr int Q = 16 / sizeof(T);
    Pad3 p3;
    size_t logical = 1;
    for (size_t d = 0; d < nd; ++d) logical *= md[d];
    // (the three-dim kernel reads the input's first element in place of one outside it: not for an empty input)
    if ((uintptr_t)out % 16 == 0 && logical > 0 && make_pad3(sp, p3))
        pad_const3_launch<T, true>(p3, in + off, out, n_out, pad_value);
    else if ((uintptr_t)out % 16 == 0)
        hipLaunchKernelGGL((pad_const_kernel<T, true, Q>), dim3(cdiv(cdiv(n_out, Q), PB)), dim3(PB), 0, stream(), sp, in + off, out, n_out, pad_value);
    else
        hipLaunchKernelGGL((pad_const_kernel<T, true, 1>), dim3(cdiv(n_out, PB)), dim3(PB), 0, stream(), sp, in + off, out, n_out, pad_value);
    MXH_LAUNCH_CHECK("pad_const");
}

// Backward of a constant pad onto a contiguous input that every output position of the interior maps to: a
// crop.  A thread owns four consecutive input elements (one vector store); `0 + g` as in the scatter form.
template <class T, int U>
__global__ __launch_bounds__(PB) void pad_crop3_kernel(Pad3 sp, const T* __restrict__ go, T* __restrict__ gi, uint32_t n_in, bool vec_store) {
    constexpr uint32_t PER = 4;
    const uint32_t base = (blockIdx.x * (uint32_t)(U * PB) + threadIdx.x) * PER;
    AVec<T, PER> v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint32_t i0 = base + (uint32_t)u * (PB * PER);
        const bool live = i0 < n_in;
        uint32_t p0, p1, p2, q;
        fd_divmod(live ? i0 : 0u, sp.in_div[2], q, p2);
        fd_divmod(q, sp.in_div[1], p0, p1);
        uint32_t row = 0;
        bool fresh = true;
#pragma unroll
        for (uint32_t e = 0; e < PER; ++e) {
            if (fresh) {
                row = (p0 + sp.before[0]) * sp.out_stride[0] + (p1 + sp.before[1]) * sp.out_stride[1] + sp.before[2];
                fresh = false;
            }
            const bool ok = live && i0 + e < n_in;           // every load is issued; position 0 of the first row stands in past the end
            v[u].v[e] = go[ok ? row + p2 : sp.before[0] * sp.out_stride[0] + sp.before[1] * sp.out_stride[1] + sp.before[2]];
            if (++p2 == sp.in[2]) {
                p2 = 0;
                fresh = true;
                if (++p1 == sp.in[1]) { p1 = 0; ++p0; }
            }
        }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const uint32_t i0 = base + (uint32_t)u * (PB * PER);
        if (i0 >= n_in) continue;
#pragma unroll
        for (uint32_t e = 0; e < PER; ++e) v[u].v[e] = PadAcc<T>::st((typename PadAcc<T>::A)0 + PadAcc<T>::ld(v[u].v[e]));
        if (vec_store && i0 + PER <= n_in) {
            *(AVec<T, PER>*)(gi + i0) = v[u];
        } else {
#pragma unroll
            for (uint32_t e = 0; e < PER; ++e)
                if (i0 + e < n_in) gi[i0 + e] = v[u].v[e];
        }
    }
}

template <class T>
void pad_backward(size_t n_in, size_t n_out, size_t nd, const size_t* md, const T* go, T* gi) {
    if (!md || !go || !gi) { set_status(ERR_INVALID, "pad_backward: null argument"); return; }
    if (n_out >= (1ull << 31)) { set_status(ERR_TOO_LARGE, "pad_backward: 2^31 or more elements"); return; }
    PadSpace sp; size_t off; bool cont, exact;
    if (!build_space(nd, md, sp, &off, &cont, &exact)) { set_status(ERR_UNSUPPORTED, "pad_backward: rank above 8 after collapse"); return; }
    // The reference writes num_els_in contiguous elements at grad_in + offset; positions no
    // output element maps to hold 0.  With a contiguous input and out = in + pads every position is hit.
    if (!(cont && exact) && n_in) {
        hipLaunchKernelGGL(zero_kernel<T>, dim3(cdiv(n_in, PB)), dim3(PB), 0, stream(), gi + off, n_in);
        MXH_LAUNCH_CHECK("pad_zero");
    }
    if (n_out == 0) return;
    constexpr int Q = 16 / sizeof(T);
    Pad3 p3;
    size_t logical = 1;
    for (size_t d = 0; d < nd; ++d) logical *= md[d];
    if (cont && exact && logical == n_in && logical > 0 && logical < (1ull << 31) && make_pad3(sp, p3)) {
        // every input position is read back from exactly one output position: gather by input element, which
        // keeps the stores whole vectors
        const bool vec_store = (uintptr_t)(gi + off) % (4 * sizeof(T)) == 0;
        if (logical >= (size_t)PB * 16 * 1024)
            hipLaunchKernelGGL((pad_crop3_kernel<T, 4>), dim3(cdiv(logical, (size_t)PB * 16)), dim3(PB), 0, stream(), p3, go, gi + off, (uint32_t)logical, vec_store);
        else
            hipLaunchKernelGGL((pad_crop3_kernel<T, 1>), dim3(cdiv(logical, (size_t)PB * 4)), dim3(PB), 0, stream(), p3, go, gi + off, (uint32_t)logical, vec_store);
        MXH_LAUNCH_CHECK("pad_const_backward");
        return;
    }
    if ((uintptr_t)go % 16 == 0 && make_pad3(sp, p3))
        pad_const3_launch<T, false>(p3, go, gi + off, n_out, T{});
    else if ((uintptr_t)go % 16 == 0)
        hipLaunchKernelGGL((pad_const_kernel<T, false, Q>), dim3(cdiv(cdiv(n_out, Q), PB)), dim3(PB), 0, stream(), sp, go, gi + off, n_out, T{});
    else
        hipLaunchKernelGGL((pad_const_kernel<T, false, 1>), dim3(cdiv(n_out, PB)), dim3(PB), 0, stream(), sp, go, gi + off, n_out, T{});
    MXH_LAUNCH_CHECK("pad_const_backward");
}

// ---- reflection and replication -----------------------------------------------------------------------
// Forward (padding.rs:115-325): every output coordinate maps to an input coordinate per dim — clamped
// (replication) or mirrored at 0 and at dim-1 until inside (reflection) — and the element is copied.
// Backward (:438-665): every input element receives the sum of the output gradients that were read
// from it.  Gather form: per dim the output coordinates that map to an input coordinate p are
// enumerated in ascending order (replication: a run; reflection: p + k*P and -p + k*P shifted by the
// leading pad, P = 2*(dim-1)), and the dims are walked like an odometer, so a thread adds its terms in
// ascending output index — the order the reference gets with one worker.  f32 accumulation.

__device__ inline uint32_t edge_pos(int mode, int64_t pos, int64_t dim) {
    if (mode == EDGE_REPLICATE) return (uint32_t)(pos < 0 ? 0 : (pos > dim - 1 ? dim - 1 : pos));
    if (pos < 0) pos = -pos;
    else if (pos >= dim) pos = 2 * dim - pos - 2;
    while (pos < 0 || pos >= dim) {
        if (pos < 0) pos = -pos;
        else pos = 2 * dim - pos - 2;
    }
    return (uint32_t)pos;
}

template <class T>
__global__ __launch_bounds__(PB) void pad_edge_kernel(PadSpace sp, int mode, const T* __restrict__ src, T* __restrict__ dst, size_t n_out) {
    size_t i = (size_t)blockIdx.x * PB + threadIdx.x;
    if (i >= n_out) return;
    uint32_t r = (uint32_t)i;
    int64_t idx = 0;
#pragma unroll
    for (int d = MAXD - 1; d >= 0; --d) {
        if (d >= sp.ndims) continue;
        uint32_t q, c;
        if (d > 0) fd_divmod(r, sp.div[d], q, c);
        else { q = 0; c = r; }
        idx += (int64_t)edge_pos(mode, (int64_t)c - (int64_t)sp.before[d], (int64_t)sp.in_dims[d]) * sp.in_strides[d];
        r = q;
    }
    dst[i] = src[idx];
}

// The same copy for at most three dims and one reflection per side (see `simple_edge_shape`): two divisions and
// 32-bit coordinates per element, four consecutive outputs of a row per thread.
__device__ __forceinline__ uint32_t edge_pos_once(int mode, uint32_t o, uint32_t before, uint32_t dim) {
    const int32_t q = (int32_t)o - (int32_t)before;
    if (mode == EDGE_REPLICATE) return (uint32_t)(q < 0 ? 0 : (q > (int32_t)dim - 1 ? (int32_t)dim - 1 : q));
    return (uint32_t)(q < 0 ? -q : (q >= (int32_t)dim ? 2 * (int32_t)dim - q - 2 : q));
}
template <class T>
__global__ __launch_bounds__(PB) void pad_edge3_kernel(Pad3 sp, int mode, const T* __restrict__ src, T* __restrict__ dst, uint32_t n_out,
                                                       bool vec_store) {
    constexpr uint32_t PER = 4;
    const uint32_t i0 = (blockIdx.x * PB + threadIdx.x) * PER;
    if (i0 >= n_out) return;
    uint32_t q, c2, c1, c0;
    fd_divmod(i0, sp.out_div[2], q, c2);
    fd_divmod(q, sp.out_div[1], c0, c1);
    int64_t row = 0;
    bool fresh = true;
    AVec<T, PER> v;
#pragma unroll
    for (uint32_t e = 0; e < PER; ++e) {
        if (i0 + e >= n_out) break;
        if (fresh) {
            row = (int64_t)edge_pos_once(mode, c0, sp.before[0], sp.in[0]) * sp.in_stride[0] +
                  (int64_t)edge_pos_once(mode, c1, sp.before[1], sp.in[1]) * sp.in_stride[1];
            fresh = false;
        }
        v.v[e] = src[row + (int64_t)edge_pos_once(mode, c2, sp.before[2], sp.in[2]) * sp.in_stride[2]];
        if (++c2 == sp.out[2]) {          // carry into the outer coordinates
            c2 = 0;
            fresh = true;
            if (++c1 == sp.out[1]) { c1 = 0; ++c0; }
        }
    }
    if (vec_store && i0 + PER <= n_out) {
        *(AVec<T, PER>*)(dst + i0) = v;
    } else {
#pragma unroll
        for (uint32_t e = 0; e < PER; ++e)
            if (i0 + e < n_out) dst[i0 + e] = v.v[e];
    }
}
static bool simple_edge_shape(const PadSpace& sp, int mode) {
    if (sp.ndims > 3) return false;
    for (int d = 0; d < sp.ndims; ++d) {
        if ((uint64_t)sp.in_dims[d] + sp.before[d] > sp.out_dims[d] || sp.in_dims[d] == 0) return false;
        const uint32_t after = sp.out_dims[d] - sp.in_dims[d] - sp.before[d];
        if (mode == EDGE_REFLECT && (sp.before[d] > sp.in_dims[d] - 1 || after > sp.in_dims[d] - 1)) return false;
    }
    return true;
}

// what the backward walk needs besides the PadSpace: how to split an input index, where an output coordinate lands
struct EdgeWalk {
    FastDiv in_div[MAXD];
    int64_t out_strides[MAXD];
};

// Ascending enumeration of the output coordinates of one dim that map to input coordinate p.
struct EdgeIter {
    int64_t a, b, hi, period;       // next candidates of the two progressions, last coordinate, step
    __device__ void init(int mode, uint32_t p, uint32_t in_dim, uint32_t out_dim, uint32_t before) {
        hi = (int64_t)out_dim - 1;
        if (mode == EDGE_REPLICATE) {
            // a run [first, last] walked with period 1; b never fires
            a = p == 0 ? 0 : (int64_t)p + before;
            int64_t last = p == in_dim - 1 ? hi : (int64_t)p + before;
            hi = last < hi ? last : hi;
            b = INT64_MAX;
            period = 1;
            return;
        }
        period = 2 * ((int64_t)in_dim - 1);
        if (period == 0) { a = 0; b = INT64_MAX; period = 1; return; }     // in_dim == 1 (no padding allowed): everything maps to 0
        // q = o - before must be congruent to p or -p modulo the period
        auto first = [&](int64_t residue) {      // smallest o >= 0 with (o - before - residue) % period == 0
            int64_t t = residue + (int64_t)before;     // o = t + k*period
            int64_t k = t >= 0 ? -(t / period) : (-t + period - 1) / period;
            return t + k * period;
        };
        a = first((int64_t)p);
        b = first(-(int64_t)p);
    }
    __device__ bool done() const { return (a < b ? a : b) > hi; }
    __device__ int64_t cur() const { return a < b ? a : b; }
    __device__ void next() {
        int64_t c = cur();
        if (a == c) a += period;
        if (b == c) b += period;
    }
};

// The dims are walked by compile-time recursion (coordinates and iterators stay in registers): dim D loops
// over the output coordinates that map to p[D], the innermost level adds one gradient.
template <class T, int D>
__device__ __forceinline__ void edge_gather(const PadSpace& sp, const EdgeWalk& w, int mode, const uint32_t (&p)[MAXD], int64_t o,
                                            const T* __restrict__ go, typename PadAcc<T>::A& acc) {
    if constexpr (D == MAXD) {
        acc = acc + PadAcc<T>::ld(go[o]);
    } else {
        if (D >= sp.ndims) { edge_gather<T, MAXD>(sp, w, mode, p, o, go, acc); return; }
        EdgeIter it;
        for (it.init(mode, p[D], sp.in_dims[D], sp.out_dims[D], sp.before[D]); !it.done(); it.next())
            edge_gather<T, D + 1>(sp, w, mode, p, o + it.cur() * w.out_strides[D], go, acc);
    }
}

template <class T>
__global__ __launch_bounds__(PB) void pad_edge_backward_kernel(PadSpace sp, EdgeWalk w, int mode, const T* __restrict__ go,
                                                                T* __restrict__ gi, size_t n_in) {
    size_t i = (size_t)blockIdx.x * PB + threadIdx.x;
    if (i >= n_in) return;
    uint32_t p[MAXD];
    int64_t dst = 0;
    {
        uint32_t r = (uint32_t)i;
#pragma unroll
        for (int d = MAXD - 1; d >= 0; --d) {
            if (d >= sp.ndims) { p[d] = 0; continue; }
            uint32_t q, c;
            if (d > 0) fd_divmod(r, w.in_div[d], q, c);
            else { q = 0; c = r; }
            p[d] = c;
            dst += (int64_t)c * sp.in_strides[d];
            r = q;
        }
    }
    typename PadAcc<T>::A acc = 0;
    edge_gather<T, 0>(sp, w, mode, p, 0, go, acc);
    gi[dst] = PadAcc<T>::st(acc);
}

// The common shape of the backward walk: at most three dims after merging and at most one reflection per side
// (pads no larger than dim - 1).  The output coordinates that map to input coordinate p of one dim are then an
// optional mirror image on the left, the run around p + before (longer than one only for a replicated border) and an
// optional mirror image on the right - ascending, so the sums keep the reference's order.  All 32-bit, no division.
struct EdgeSrc {
    uint32_t cl, a0, a1, cr, has_l, n;
    __device__ void init(int mode, uint32_t p, uint32_t in_dim, uint32_t out_dim, uint32_t before) {
        const uint32_t after = out_dim - in_dim - before;
        a0 = a1 = p + before;
        cl = cr = 0;
        has_l = 0;
        uint32_t has_r = 0;
        if (mode == EDGE_REPLICATE) {
            if (p == 0) a0 = 0;
            if (p == in_dim - 1) a1 = out_dim - 1;
        } else if (mode == EDGE_REFLECT) {
            if (p >= 1 && p <= before) { has_l = 1; cl = before - p; }
            if (p + 1 < in_dim && p + after + 1 >= in_dim) { has_r = 1; cr = before + 2 * (in_dim - 1) - p; }
        }
        n = has_l + (a1 - a0 + 1) + has_r;
    }
    __device__ uint32_t at(uint32_t k) const {
        if (k < has_l) return cl;
        k -= has_l;
        return k <= a1 - a0 ? a0 + k : cr;
    }
};

// A thread owns four consecutive input elements; with a contiguous input they leave as one vector.
template <class T>
__global__ __launch_bounds__(PB) void pad_edge_backward3_kernel(Pad3 sp, int mode, const T* __restrict__ go, T* __restrict__ gi, uint32_t n_in,
                                                                 bool vec_store) {
    constexpr uint32_t PER = 4;
    const uint32_t i0 = (blockIdx.x * PB + threadIdx.x) * PER;
    if (i0 >= n_in) return;
    uint32_t p0, p1, p2, q;
    fd_divmod(i0, sp.in_div[2], q, p2);
    fd_divmod(q, sp.in_div[1], p0, p1);
    EdgeSrc s0, s1;
    int64_t row = 0;
    bool fresh = true;
    AVec<T, PER> v;
    int64_t dst[PER];
#pragma unroll
    for (uint32_t e = 0; e < PER; ++e) {
        if (i0 + e >= n_in) break;
        if (fresh) {
            s0.init(mode, p0, sp.in[0], sp.out[0], sp.before[0]);
            s1.init(mode, p1, sp.in[1], sp.out[1], sp.before[1]);
            row = (int64_t)p0 * sp.in_stride[0] + (int64_t)p1 * sp.in_stride[1];
            fresh = false;
        }
        EdgeSrc s2;
        s2.init(mode, p2, sp.in[2], sp.out[2], sp.before[2]);
        typename PadAcc<T>::A acc = 0;
        for (uint32_t k0 = 0; k0 < s0.n; ++k0) {
            const uint32_t o0 = s0.at(k0) * sp.out_stride[0];
            for (uint32_t k1 = 0; k1 < s1.n; ++k1) {
                const uint32_t o1 = o0 + s1.at(k1) * sp.out_stride[1];
                for (uint32_t k2 = 0; k2 < s2.n; ++k2) acc = acc + PadAcc<T>::ld(go[o1 + s2.at(k2)]);
            }
        }
        v.v[e] = PadAcc<T>::st(acc);
        dst[e] = row + (int64_t)p2 * sp.in_stride[2];
        if (++p2 == sp.in[2]) {
            p2 = 0;
            fresh = true;
            if (++p1 == sp.in[1]) { p1 = 0; ++p0; }
        }
    }
    if (vec_store && i0 + PER <= n_in) {
        *(AVec<T, PER>*)(gi + i0) = v;
    } else {
#pragma unroll
        for (uint32_t e = 0; e < PER; ++e)
            if (i0 + e < n_in) gi[dst[e]] = v.v[e];
    }
}

// The input coordinates of one dim that receive more than one output gradient ("special"): for a reflection those a
// mirror image lands on (1 .. before on the left, in-1-after .. in-2 on the right), for a replication the two ends when
// their side is padded.  Everything else receives exactly the gradient at p + before.
struct SpecialSet {
    uint32_t nl, l0, nr, r0;
    __host__ __device__ uint32_t size() const { return nl + nr; }
    __host__ __device__ uint32_t at(uint32_t k) const { return k < nl ? l0 + k : r0 + (k - nl); }
};
static SpecialSet special_set(int mode, uint32_t in_dim, uint32_t out_dim, uint32_t before) {
    const uint32_t after = out_dim - in_dim - before;
    SpecialSet s{0, 0, 0, 0};
    if (mode == EDGE_REPLICATE) {
        if (before) { s.nl = 1; s.l0 = 0; }
        if (after) { s.nr = 1; s.r0 = in_dim - 1; }
    } else {
        s.nl = before; s.l0 = 1;
        s.nr = after; s.r0 = in_dim - 1 - after;
    }
    return s;
}
struct SpecialSets {
    SpecialSet d[3];
    uint32_t count[3];        // elements of the box in which dim k runs over its special coordinates
    __host__ __device__ static bool has(const SpecialSet& s, uint32_t p) { return p - s.l0 < s.nl || p - s.r0 < s.nr; }
};
// One launch, two classes of blocks, so that no wave meets both kinds of work.
// The first `walk_blocks` blocks (first, so that their longer work starts early and the copy fills in around it): one
// thread per element of the rows whose coordinate in dim 0 or in dim 1 is special (whole rows, so their stores are
// contiguous), the full sum in the reference's order; a row special in both dims is written twice, with the same values.
// The other blocks: a thread owns four consecutive input elements of the other rows and gives each its one gradient, the
// one at p + before (vector loads of whole rows, vector stores); an element special in the last dim only - two or so per
// row - gets the few gradients of its own output row instead.
template <class T>
__global__ __launch_bounds__(PB) void pad_edge_backward_split_kernel(Pad3 sp, int mode, SpecialSets sets, uint32_t walk_blocks, const T* __restrict__ go,
                                                                     T* __restrict__ gi, uint32_t n_in, bool vec_store) {
    constexpr uint32_t PER = 4;
    if (blockIdx.x >= walk_blocks) {
        const uint32_t i0 = ((blockIdx.x - walk_blocks) * PB + threadIdx.x) * PER;
        if (i0 >= n_in) return;
        uint32_t p0, p1, p2, q;
        fd_divmod(i0, sp.in_div[2], q, p2);
        fd_divmod(q, sp.in_div[1], p0, p1);
        uint32_t row = 0;
        bool fresh = true, row_special = false;
        AVec<T, PER> v;
        uint32_t skip = 0, walk = 0;
        uint32_t rows[PER], cols[PER];
#pragma unroll
        for (uint32_t e = 0; e < PER; ++e) {
            if (fresh) {
                row = (p0 + sp.before[0]) * sp.out_stride[0] + (p1 + sp.before[1]) * sp.out_stride[1];
                row_special = SpecialSets::has(sets.d[0], p0) || SpecialSets::has(sets.d[1], p1);
                fresh = false;
            }
            const bool ok = i0 + e < n_in;
            if (!ok || row_special) skip |= 1u << e;
            else if (SpecialSets::has(sets.d[2], p2)) walk |= 1u << e;
            rows[e] = row;
            cols[e] = p2;
            v.v[e] = go[ok ? row + sp.before[2] + p2 : sp.before[0] * sp.out_stride[0] + sp.before[1] * sp.out_stride[1] + sp.before[2]];
            if (++p2 == sp.in[2]) {
                p2 = 0;
                fresh = true;
                if (++p1 == sp.in[1]) { p1 = 0; ++p0; }
            }
        }
#pragma unroll
        for (uint32_t e = 0; e < PER; ++e) {
            typename PadAcc<T>::A acc = 0;
            if (walk & (1u << e)) {
                // special in the last dim only: the few gradients of its own output row, in ascending order
                EdgeSrc s2;
                s2.init(mode, cols[e], sp.in[2], sp.out[2], sp.before[2]);
                for (uint32_t k2 = 0; k2 < s2.n; ++k2) acc = acc + PadAcc<T>::ld(go[rows[e] + s2.at(k2)]);
            } else {
                acc = acc + PadAcc<T>::ld(v.v[e]);
            }
            v.v[e] = PadAcc<T>::st(acc);
        }
        if (vec_store && skip == 0) {
            *(AVec<T, PER>*)(gi + i0) = v;
        } else {
#pragma unroll
            for (uint32_t e = 0; e < PER; ++e)
                if (!(skip & (1u << e))) gi[i0 + e] = v.v[e];
        }
        return;
    }
    uint32_t t = blockIdx.x * PB + threadIdx.x;
    int D = 0;
    if (t >= sets.count[0]) { t -= sets.count[0]; D = 1; if (t >= sets.count[1]) return; }
    // the box: dim D runs over the special coordinates, the others over the whole input; the last dim moves fastest
    const uint32_t e1 = D == 1 ? sets.d[1].size() : sp.in[1], e2 = sp.in[2];
    uint32_t p2 = t % e2, q = t / e2;
    uint32_t p1 = q % e1, p0 = q / e1;
    if (D == 0) p0 = sets.d[0].at(p0);
    else p1 = sets.d[1].at(p1);
    EdgeSrc s0, s1, s2;
    s0.init(mode, p0, sp.in[0], sp.out[0], sp.before[0]);
    s1.init(mode, p1, sp.in[1], sp.out[1], sp.before[1]);
    s2.init(mode, p2, sp.in[2], sp.out[2], sp.before[2]);
    typename PadAcc<T>::A acc = 0;
    for (uint32_t k0 = 0; k0 < s0.n; ++k0) {
        const uint32_t o0 = s0.at(k0) * sp.out_stride[0];
        for (uint32_t k1 = 0; k1 < s1.n; ++k1) {
            const uint32_t o1 = o0 + s1.at(k1) * sp.out_stride[1];
            for (uint32_t k2 = 0; k2 < s2.n; ++k2) acc = acc + PadAcc<T>::ld(go[o1 + s2.at(k2)]);
        }
    }
    gi[(int64_t)p0 * sp.in_stride[0] + (int64_t)p1 * sp.in_stride[1] + (int64_t)p2 * sp.in_stride[2]] = PadAcc<T>::st(acc);
}

static bool edge_space(size_t nd_full, const size_t* md_full, int mode, PadSpace& sp, EdgeWalk& in_walk, size_t* in_off, const char* who) {
    if (nd_full > 64) { set_status(ERR_UNSUPPORTED, who); return false; }
    *in_off = md_full[2 * nd_full];
    // Merge runs of dims without padding whose input strides chain (they map to themselves), so that
    // [B, C, H, W] padded on H and W walks three dims.
    size_t in_dims[64], st_m[64], out_dims[64], pads[128];
    size_t nd = 0;
    {
        const size_t* fin = md_full;
        const size_t* fst = md_full + nd_full;
        const size_t* fout = md_full + 2 * nd_full + 1;
        const size_t* fp = md_full + 3 * nd_full + 1;
        bool cont = ref_is_contiguous(nd_full, fin, fst);
        size_t cs[64];
        contiguous_strides(nd_full, fin, cs);
        const size_t* st = cont ? cs : fst;       // padding.rs:199-214: contiguous inputs are indexed row-major
        for (size_t d = 0; d < nd_full; ++d) {
            bool plain = fp[2 * d] == 0 && fout[d] == fin[d];
            if (plain && fin[d] == 1) continue;
            if (nd > 0 && plain && pads[2 * (nd - 1)] == 0 && out_dims[nd - 1] == in_dims[nd - 1] && st_m[nd - 1] == st[d] * fin[d]) {
                in_dims[nd - 1] *= fin[d]; out_dims[nd - 1] *= fout[d]; st_m[nd - 1] = st[d];
            } else {
                in_dims[nd] = fin[d]; out_dims[nd] = fout[d]; st_m[nd] = st[d]; pads[2 * nd] = fp[2 * d]; pads[2 * nd + 1] = fp[2 * d + 1]; ++nd;
            }
        }
    }
    if (nd > (size_t)MAXD) { set_status(ERR_UNSUPPORTED, who); return false; }
    const size_t* st = st_m;
    sp.ndims = (int)(nd ? nd : 1);
    int64_t ost = 1;
    for (int d = MAXD - 1; d >= 0; --d) {
        in_walk.out_strides[d] = d < (int)nd ? ost : 0;
        if (d < (int)nd) ost *= (int64_t)out_dims[d];
    }
    for (int d = 0; d < MAXD; ++d) {
        bool real = d < (int)nd;
        if (real && (in_dims[d] >= (1ull << 31) || out_dims[d] >= (1ull << 31) || pads[2 * d] >= (1ull << 31))) { set_status(ERR_TOO_LARGE, who); return false; }
        if (real && in_dims[d] == 0 && out_dims[d] != 0) { set_status(ERR_INVALID, who); return false; }
        // the reference's mirror loop never ends for a padded dim of size 1
        if (real && mode == EDGE_REFLECT && in_dims[d] == 1 && out_dims[d] != 1) { set_status(ERR_INVALID, "pad_with_reflection: a dim of size 1 cannot be mirrored"); return false; }
        sp.out_dims[d] = real ? (uint32_t)out_dims[d] : 1;
        sp.in_dims[d] = real ? (uint32_t)in_dims[d] : 1;
        sp.before[d] = real ? (uint32_t)pads[2 * d] : 0;
        sp.in_strides[d] = real ? (int64_t)st[d] : 0;
        sp.div[d] = make_fastdiv(sp.out_dims[d]);
        in_walk.in_div[d] = make_fastdiv(sp.in_dims[d]);
    }
    sp.out_last = sp.in_last = 1; sp.before_last = 0; sp.stride_last = 0; sp.div_last = make_fastdiv(1);
    return true;
}

template <class T>
void pad_edge_forward(int mode, size_t n_in, size_t n_out, size_t nd, const size_t* md, const T* in, T* out) {
    (void)n_in;
    if (!md || !in || !out) { set_status(ERR_INVALID, "pad: null argument"); return; }
    if (n_out == 0) return;
    if (n_out >= (1ull << 31)) { set_status(ERR_TOO_LARGE, "pad: output of 2^31 or more elements"); return; }
    PadSpace sp; EdgeWalk walk; size_t off;
    if (!edge_space(nd, md, mode, sp, walk, &off, "pad_with_reflection/replication: bad shape or rank above 8")) return;
    Pad3 p3;
    if (simple_edge_shape(sp, mode) && make_pad3(sp, p3))
        hipLaunchKernelGGL(pad_edge3_kernel<T>, dim3(cdiv(n_out, (size_t)PB * 4)), dim3(PB), 0, stream(), p3, mode, in + off, out, (uint32_t)n_out,
                           (uintptr_t)out % (4 * sizeof(T)) == 0);
    else
        hipLaunchKernelGGL(pad_edge_kernel<T>, dim3(cdiv(n_out, PB)), dim3(PB), 0, stream(), sp, mode, in + off, out, n_out);
    MXH_LAUNCH_CHECK("pad_edge");
}

template <class T>
void pad_edge_backward(int mode, size_t n_in, size_t n_out, size_t nd, const size_t* md, const T* go, T* gi) {
    if (!md || !go || !gi) { set_status(ERR_INVALID, "pad_backward: null argument"); return; }
    if (n_in == 0) return;
    if (n_out >= (1ull << 31) || n_in >= (1ull << 31)) { set_status(ERR_TOO_LARGE, "pad_backward: 2^31 or more elements"); return; }
    PadSpace sp; EdgeWalk walk; size_t off;
    if (!edge_space(nd, md, mode, sp, walk, &off, "pad_with_reflection/replication backward: bad shape or rank above 8")) return;
    // the reference writes num_els_in contiguous elements at grad_in + offset: positions a strided
    // layout does not reach hold 0
    bool cont = ref_is_contiguous(nd, md, md + nd);
    if (!cont) {
        hipLaunchKernelGGL(zero_kernel<T>, dim3(cdiv(n_in, PB)), dim3(PB), 0, stream(), gi + off, n_in);
        MXH_LAUNCH_CHECK("pad_zero");
    }
    size_t logical = 1;
    for (size_t d = 0; d < nd; ++d) logical *= md[d];
    if (logical == 0) return;
    Pad3 p3;
    const bool simple = simple_edge_shape(sp, mode) && make_pad3(sp, p3);
    if (simple && cont && logical == n_in && logical >= (size_t)PB * 64 && logical < (1ull << 31)) {
        // Large and contiguous: all but a thin border of the input receives exactly one gradient, the one at p + before.
        // A kernel that tests per element spends a whole wave's time on the walk wherever one lane meets the border,
        // which is in every wave once rows are shorter than a wave's 256 elements; here the copy and the walk are done by
        // different blocks of one launch.
        SpecialSets sets;
        size_t border = 0;
        for (int d = 0; d < 3; ++d) {
            sets.d[d] = special_set(mode, p3.in[d], p3.out[d], p3.before[d]);
            size_t count = sets.d[d].size();
            for (int k = 0; k < 3; ++k)
                if (k != d) count *= p3.in[k];
            sets.count[d] = (uint32_t)count;
            if (d < 2) border += count;
        }
        const uint32_t copy_blocks = (uint32_t)cdiv(logical, (size_t)PB * 4), walk_blocks = (uint32_t)cdiv(border, (size_t)PB);
        hipLaunchKernelGGL(pad_edge_backward_split_kernel<T>, dim3(copy_blocks + walk_blocks), dim3(PB), 0, stream(), p3, mode, sets,
                           walk_blocks, go, gi + off, (uint32_t)logical, (uintptr_t)(gi + off) % (4 * sizeof(T)) == 0);
        MXH_LAUNCH_CHECK("pad_edge_backward_split");
        return;
    }
    if (simple)
        hipLaunchKernelGGL(pad_edge_backward3_kernel<T>, dim3(cdiv(logical, (size_t)PB * 4)), dim3(PB), 0, stream(), p3, mode, go, gi + off, (uint32_t)logical,
                           cont && (uintptr_t)(gi + off) % (4 * sizeof(T)) == 0);
    else
        hipLaunchKernelGGL(pad_edge_backward_kernel<T>, dim3(cdiv(logical, PB)), dim3(PB), 0, stream(), sp, walk, mode, go, gi + off, logical);
    MXH_LAUNCH_CHECK("pad_edge_backward");
}

}  // namespace mxh

using namespace mxh;

#define MXH_PAD_FOR(T, SUF)                                                                                  \
    extern "C" void hip_pad_with_constant_##SUF(size_t n_in, size_t n_out, size_t nd, const size_t* md,      \
                                                const T* in, T* out, T pad_value) { MXH_API;                 \
        pad_forward<T>(n_in, n_out, nd, md, in, out, pad_value);                                             \
    }                                                                                                        \
    extern "C" void hip_pad_with_constant_backward_##SUF(size_t n_in, size_t n_out, size_t nd,               \
                                                         const size_t* md, const T* go, T* gi) { MXH_API;    \
        pad_backward<T>(n_in, n_out, nd, md, go, gi);                                                        \
    }

#define MXH_PAD_EDGE_FOR(T, SUF)                                                                             \
    extern "C" void hip_pad_with_reflection_##SUF(size_t n_in, size_t n_out, size_t nd, const size_t* md,    \
                                                  const T* in, T* out) { MXH_API;                            \
        pad_edge_forward<T>(EDGE_REFLECT, n_in, n_out, nd, md, in, out);                                     \
    }                                                                                                        \
    extern "C" void hip_pad_with_replication_##SUF(size_t n_in, size_t n_out, size_t nd, const size_t* md,   \
                                                   const T* in, T* out) { MXH_API;                           \
        pad_edge_forward<T>(EDGE_REPLICATE, n_in, n_out, nd, md, in, out);                                   \
    }                                                                                                        \
    extern "C" void hip_pad_with_reflection_backward_##SUF(size_t n_in, size_t n_out, size_t nd,             \
                                                           const size_t* md, const T* go, T* gi) { MXH_API;  \
        pad_edge_backward<T>(EDGE_REFLECT, n_in, n_out, nd, md, go, gi);                                     \
    }                                                                                                        \
    extern "C" void hip_pad_with_replication_backward_##SUF(size_t n_in, size_t n_out, size_t nd,            \
                                                            const size_t* md, const T* go, T* gi) { MXH_API; \
        pad_edge_backward<T>(EDGE_REPLICATE, n_in, n_out, nd, md, go, gi);                                   \
    }

MXH_PAD_EDGE_FOR(float, f32)
MXH_PAD_EDGE_FOR(bf16_t, bf16)
MXH_PAD_EDGE_FOR(f16_t, f16)
MXH_PAD_FOR(float, f32)
MXH_PAD_FOR(bf16_t, bf16)
MXH_PAD_FOR(f16_t, f16)
MXH_PAD_EDGE_FOR(double, f64)      // (crates/maidenx_cuda/src/ops/padding.rs:82)
MXH_PAD_FOR(double, f64)
// the integers (crates/maidenx_cuda/src/ops/padding.rs:83-90)
#define MXH_PAD_INT(T, SUF) MXH_PAD_EDGE_FOR(T, SUF) MXH_PAD_FOR(T, SUF)
MXH_PAD_INT(uint8_t, u8)
MXH_PAD_INT(uint16_t, u16)
MXH_PAD_INT(uint32_t, u32)
MXH_PAD_INT(uint64_t, u64)
MXH_PAD_INT(int8_t, i8)
MXH_PAD_INT(int16_t, i16)
MXH_PAD_INT(int32_t, i32)
MXH_PAD_INT(int64_t, i64)
