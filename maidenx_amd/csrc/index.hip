// Index ops on the device: index_select, index_add_, gather, scatter_add_, bincount.
// The reference has no backend symbol for these: crates/maidenx_tensor/src/ops/indexing.rs runs them
// as host loops over `get` / `set` / `add_at_index` (one buffer round trip per element).  The entry
// points here take the tensors' layouts (dims[n] | strides[n] | offset, as the tensor layer holds
// them) and do the same work in one launch, with the same results:
//   index_select (:93-124)  out[.., i, ..] = in[.., idx[i], ..]            copy, bit-exact
//   gather       (:315-363) out[p] = in[p with p[dim] = index[p]]         copy, bit-exact; negative wraps
//   index_add_   (:15-91)   self[.., idx[i], ..] += src[.., i, ..]         i ascending
//   scatter_add_ (:403-461) self[p with p[dim] = index[p]] += src[p]       p in row-major order
//   bincount     (:463-522) counts, or sums of weights, per value
// The adds are in the storage dtype (utils/indexing.rs:96-140) and their order matters for floats.
// Updates of different "lines" (all coordinates but `dim` fixed) never meet, and inside a line the
// reference's order is ascending position along `dim`: one thread owns a line and walks it in that
// order, so results are bit-identical to the host loops and deterministic.  Counts are integers
// (atomics are exact); weighted bincount lets one thread own a bin and scan the input in order.
// index_add_ with many indices sorts them by destination first (stable), see below.
// An index outside its range is skipped and raises the device-side index flag, which
// hip_get_last_status() reports as an invalid argument (the reference returns IndexOutOfBounds).
#include <cstring>


#include "elementwise.hpp"
#include "mxh.hpp"
#include "radix_sort.hpp"
#include "ops.hpp"

namespace mxh {

constexpr int IB = 256;

// add_at_index (crates/maidenx_tensor/src/utils/indexing.rs:121-135): `+` in the storage dtype.  The floats round per
// add (Ar<T>::add), bool is `||` (its Ar<T>::add), the integers wrap (the reference's release build; the saturating add
// of the binary op family is a different function).
template <class T> __device__ inline T idx_add(T a, T b) {
    if constexpr (std::is_integral<T>::value) {
        using U = typename std::make_unsigned<T>::type;
        return (T)(U)((U)a + (U)b);
    } else return Ar<T>::add(a, b);
}

struct Lay {            // one tensor: shape walk + strides
    int64_t strides[MAXD];
    int64_t offset;
};
struct IdxSpace {
    int nd, dim;
    uint32_t dims[MAXD];        // iteration space
    FastDiv div[MAXD];
};

// decompose a linear index over the iteration space into coordinates (row-major)
__device__ inline void split(const IdxSpace& sp, uint32_t r, uint32_t (&c)[MAXD]) {
#pragma unroll
    for (int d = MAXD - 1; d >= 0; --d) {
        if (d >= sp.nd) { c[d] = 0; continue; }
        uint32_t q, m;
        if (d > 0) fd_divmod(r, sp.div[d], q, m);
        else { q = 0; m = r; }
        c[d] = m;
        r = q;
    }
}
__device__ inline int64_t dot(const IdxSpace& sp, const uint32_t (&c)[MAXD], const Lay& l, int skip_dim) {
    int64_t o = l.offset;
#pragma unroll
    for (int d = 0; d < MAXD; ++d)
        if (d < sp.nd && d != skip_dim) o += (int64_t)c[d] * l.strides[d];
    return o;
}

// ---- index_select: iteration space = output dims ------------------------------------------------
template <class T, class I>
__global__ __launch_bounds__(IB) void index_select_kernel(IdxSpace sp, Lay in, const I* __restrict__ indices, int64_t idx_stride,
                                                          int64_t idx_offset, uint32_t in_dim_size, const T* __restrict__ src,
                                                          T* __restrict__ out, size_t n, int* flag) {
    size_t o = (size_t)blockIdx.x * IB + threadIdx.x;
    if (o >= n) return;
    uint32_t c[MAXD];
    split(sp, (uint32_t)o, c);
    // the reference reads the index `as_i32` (:113)
    const int32_t idx = (int32_t)indices[idx_offset + (int64_t)c[sp.dim] * idx_stride];
    if (idx < 0 || (uint32_t)idx >= in_dim_size) { *flag = 1; out[o] = T{}; return; }
    out[o] = src[dot(sp, c, in, sp.dim) + (int64_t)idx * in.strides[sp.dim]];
}

// contiguous input seen as [outer, D, inner] with inner a multiple of the 16-byte vector: rows move as vectors
template <class T, class I, int VEC>
__global__ __launch_bounds__(IB) void index_select_rows_kernel(const I* __restrict__ indices, int64_t idx_stride, int64_t idx_offset,
                                                               uint32_t n_idx, uint32_t D, uint32_t inner_v, FastDiv div_inner,
                                                               FastDiv div_nidx, const T* __restrict__ src, T* __restrict__ out,
                                                               size_t nvec, int* flag) {
    struct alignas(16) V { T v[VEC]; };
    size_t o = (size_t)blockIdx.x * IB + threadIdx.x;
    if (o >= nvec) return;
    uint32_t r, v, outer, i;
    fd_divmod((uint32_t)o, div_inner, r, v);
    fd_divmod(r, div_nidx, outer, i);
    const int32_t idx = (int32_t)indices[idx_offset + (int64_t)i * idx_stride];
    V val;
    if (idx < 0 || (uint32_t)idx >= D) {
        *flag = 1;
#pragma unroll
        for (int e = 0; e < VEC; ++e) val.v[e] = T{};
    } else {
        val = *(const V*)(src + (((size_t)outer * D + (uint32_t)idx) * inner_v + v) * VEC);
    }
    *(V*)(out + o * VEC) = val;
}

// ---- gather: iteration space = index dims ---------------------------------------------------------
template <class T, class I>
__global__ __launch_bounds__(IB) void gather_kernel(IdxSpace sp, Lay in, Lay ix, uint32_t in_dim_size, const I* __restrict__ index,
                                                    const T* __restrict__ src, T* __restrict__ out, size_t n, int* flag) {
    size_t o = (size_t)blockIdx.x * IB + threadIdx.x;
    if (o >= n) return;
    uint32_t c[MAXD];
    split(sp, (uint32_t)o, c);
    int32_t idx = (int32_t)index[dot(sp, c, ix, -1)];
    if (idx < 0) idx += (int32_t)in_dim_size;              // :341-345
    if (idx < 0 || (uint32_t)idx >= in_dim_size) { *flag = 1; out[o] = T{}; return; }
    out[o] = src[dot(sp, c, in, sp.dim) + (int64_t)idx * in.strides[sp.dim]];
}

// ---- index_add_ / scatter_add_: iteration space = the lines (dims[dim] forced to 1) ----------------
template <class T, class I>
__global__ __launch_bounds__(IB) void index_add_kernel(IdxSpace sp, Lay self, Lay sr, const I* __restrict__ indices, int64_t idx_stride,
                                                       int64_t idx_offset, uint32_t n_idx, uint32_t self_dim_size,
                                                       const T* __restrict__ src, T* __restrict__ dst, size_t lines, int* flag) {
    size_t l = (size_t)blockIdx.x * IB + threadIdx.x;
    if (l >= lines) return;
    uint32_t c[MAXD];
    split(sp, (uint32_t)l, c);
    const int64_t s0 = dot(sp, c, sr, sp.dim), d0 = dot(sp, c, self, sp.dim);
    for (uint32_t i = 0; i < n_idx; ++i) {
        const int32_t idx = (int32_t)indices[idx_offset + (int64_t)i * idx_stride];
        if (idx < 0 || (uint32_t)idx >= self_dim_size) { *flag = 1; continue; }
        T* p = dst + d0 + (int64_t)idx * self.strides[sp.dim];
        *p = idx_add<T>(*p, src[s0 + (int64_t)i * sr.strides[sp.dim]]);
    }
}

// Many indices, few lines (an embedding gradient): the indices are sorted by destination with a stable
// radix sort (radix_sort.hpp; equal destinations keep ascending i), and one thread per destination
// element adds its sources in that order — the same order as the walk above, with parallelism over
// the whole of self instead of over the lines.
template <class I>
__global__ __launch_bounds__(IB) void index_keys_kernel(const I* __restrict__ indices, int64_t idx_stride, int64_t idx_offset, uint32_t n_idx,
                                                        uint32_t self_dim_size, uint32_t* keys, uint32_t* vals, int* flag) {
    uint32_t i = blockIdx.x * IB + threadIdx.x;
    if (i >= n_idx) return;
    const int32_t idx = (int32_t)indices[idx_offset + (int64_t)i * idx_stride];
    const bool ok = idx >= 0 && (uint32_t)idx < self_dim_size;
    if (!ok) *flag = 1;
    keys[i] = ok ? (uint32_t)idx : self_dim_size;       // out of range: sorted behind every real destination, never applied
    vals[i] = i;
}

template <class T>
__global__ __launch_bounds__(IB) void index_add_sorted_kernel(IdxSpace sp, Lay self, Lay sr, const uint32_t* __restrict__ keys,
                                                              const uint32_t* __restrict__ vals, uint32_t n_idx, uint32_t lines,
                                                              FastDiv div_lines, const T* __restrict__ src, T* __restrict__ dst,
                                                              size_t work) {
    size_t wi = (size_t)blockIdx.x * IB + threadIdx.x;
    if (wi >= work) return;
    uint32_t d, l;
    fd_divmod((uint32_t)wi, div_lines, d, l);
    // first entry with key >= d
    uint32_t lo = 0, hi = n_idx;
    while (lo < hi) {
        uint32_t mid = (lo + hi) >> 1;
        if (keys[mid] < d) lo = mid + 1;
        else hi = mid;
    }
    if (lo >= n_idx || keys[lo] != d) return;
    uint32_t c[MAXD];
    split(sp, l, c);
    const int64_t s0 = dot(sp, c, sr, sp.dim);
    T* p = dst + dot(sp, c, self, sp.dim) + (int64_t)d * self.strides[sp.dim];
    T acc = *p;
    for (uint32_t k = lo; k < n_idx && keys[k] == d; ++k) acc = idx_add<T>(acc, src[s0 + (int64_t)vals[k] * sr.strides[sp.dim]]);
    *p = acc;
}

// the same for contiguous self [outer, D, inner] and src [outer, n_idx, inner] with inner a multiple of the
// 16-byte vector: a block owns (outer, destination row, 256 vectors of the row) and searches once
template <class T, int VEC>
__global__ __launch_bounds__(IB) void index_add_rows_kernel(const uint32_t* __restrict__ keys, const uint32_t* __restrict__ vals, uint32_t n_idx,
                                                            uint32_t D, uint32_t inner_v, uint32_t chunks, FastDiv div_chunks, FastDiv div_D,
                                                            const T* __restrict__ src, T* __restrict__ dst) {
    struct alignas(16) V { T v[VEC]; };
    uint32_t r, chunk, outer, d;
    fd_divmod(blockIdx.x, div_chunks, r, chunk);
    fd_divmod(r, div_D, outer, d);
    uint32_t lo = 0, hi = n_idx;
    while (lo < hi) {
        uint32_t mid = (lo + hi) >> 1;
        if (keys[mid] < d) lo = mid + 1;
        else hi = mid;
    }
    if (lo >= n_idx || keys[lo] != d) return;
    const uint32_t v = chunk * IB + threadIdx.x;
    if (v >= inner_v) return;
    V* p = (V*)(dst + (((size_t)outer * D + d) * inner_v + v) * VEC);
    V acc = *p;
    for (uint32_t k = lo; k < n_idx && keys[k] == d; ++k) {
        const V s = *(const V*)(src + (((size_t)outer * n_idx + vals[k]) * inner_v + v) * VEC);
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc.v[e] = idx_add<T>(acc.v[e], s.v[e]);
    }
    *p = acc;
}

template <class T, class I>
__global__ __launch_bounds__(IB) void scatter_add_kernel(IdxSpace sp, Lay self, Lay ix, Lay sr, uint32_t len, uint32_t self_dim_size,
                                                         const I* __restrict__ index, const T* __restrict__ src, T* __restrict__ dst,
                                                         size_t lines, int* flag) {
    size_t l = (size_t)blockIdx.x * IB + threadIdx.x;
    if (l >= lines) return;
    uint32_t c[MAXD];
    split(sp, (uint32_t)l, c);
    const int64_t s0 = dot(sp, c, sr, sp.dim), i0 = dot(sp, c, ix, sp.dim), d0 = dot(sp, c, self, sp.dim);
    for (uint32_t k = 0; k < len; ++k) {
        int32_t idx = (int32_t)index[i0 + (int64_t)k * ix.strides[sp.dim]];
        if (idx < 0) idx += (int32_t)self_dim_size;          // :434-438
        if (idx < 0 || (uint32_t)idx >= self_dim_size) { *flag = 1; continue; }
        T* p = dst + d0 + (int64_t)idx * self.strides[sp.dim];
        *p = idx_add<T>(*p, src[s0 + (int64_t)k * sr.strides[sp.dim]]);
    }
}

// ---- bincount ---------------------------------------------------------------------------------------
template <class I>
__global__ __launch_bounds__(IB) void zero_counts_kernel(I* out, size_t n) {
    size_t i = (size_t)blockIdx.x * IB + threadIdx.x;
    if (i < n) out[i] = 0;
}
template <class I> __device__ inline void count_one(I* p);
template <> __device__ inline void count_one<int32_t>(int32_t* p) { atomicAdd(p, 1); }
template <> __device__ inline void count_one<int64_t>(int64_t* p) { atomicAdd((unsigned long long*)p, 1ull); }

template <class I>
__global__ __launch_bounds__(IB) void bincount_kernel(const I* __restrict__ in, int64_t stride, int64_t offset, size_t n, I* out,
                                                      size_t out_size, int* flag) {
    size_t i = (size_t)blockIdx.x * IB + threadIdx.x;
    if (i >= n) return;
    const int32_t v = (int32_t)in[offset + (int64_t)i * stride];
    if (v < 0 || (size_t)v >= out_size) { *flag = 1; return; }
    count_one<I>(out + v);
}
// one thread per bin, input scanned in order: sum of the weights of the entries equal to the bin
template <class T, class I>
__global__ __launch_bounds__(IB) void bincount_weighted_kernel(const I* __restrict__ in, int64_t stride, int64_t offset,
                                                               const T* __restrict__ w, int64_t w_stride, int64_t w_offset, size_t n,
                                                               T* out, size_t out_size, int* flag) {
    size_t b = (size_t)blockIdx.x * IB + threadIdx.x;
    if (b >= out_size) return;
    T acc = Ar<T>::zero();
    for (size_t i = 0; i < n; ++i) {
        const int32_t v = (int32_t)in[offset + (int64_t)i * stride];
        if (b == 0 && (v < 0 || (size_t)v >= out_size)) *flag = 1;
        if (v >= 0 && (size_t)v == b) acc = idx_add<T>(acc, w[w_offset + (int64_t)i * w_stride]);
    }
    out[b] = acc;
}

// ---- host side ----------------------------------------------------------------------------------------
// layout = dims[n] | strides[n] | offset
static bool read_layout(size_t nd, const size_t* layout, Lay& l) {
    for (int d = 0; d < MAXD; ++d) l.strides[d] = d < (int)nd ? (int64_t)layout[nd + d] : 0;
    l.offset = (int64_t)layout[2 * nd];
    return true;
}
// iteration space over `dims` with dims[force_one] treated as 1 when force_one >= 0
static bool make_space(size_t nd, const size_t* dims, size_t dim, int force_one, IdxSpace& sp, size_t* count, const char* who) {
    if (nd == 0 || nd > (size_t)MAXD || dim >= nd) { set_status(ERR_INVALID, who); return false; }
    sp.nd = (int)nd;
    sp.dim = (int)dim;
    size_t total = 1;
    for (int d = 0; d < MAXD; ++d) {
        size_t v = d < (int)nd ? dims[d] : 1;
        if (d == force_one) v = 1;
        if (v >= (1ull << 31)) { set_status(ERR_TOO_LARGE, who); return false; }
        sp.dims[d] = (uint32_t)v;
        sp.div[d] = make_fastdiv((uint32_t)v);
        total *= v;
    }
    if (total >= (1ull << 31)) { set_status(ERR_TOO_LARGE, who); return false; }
    *count = total;
    return true;
}

template <class T, class I>
void index_select(size_t nd, size_t dim, const size_t* in_layout, size_t n_idx, size_t idx_stride, size_t idx_offset, const I* indices,
                  const T* input, T* output) {
    if (!in_layout || !indices || !input || !output) { set_status(ERR_INVALID, "index_select: null argument"); return; }
    int* flag = index_flag();
    if (!flag) return;
    size_t out_dims[MAXD];
    if (nd > (size_t)MAXD || dim >= nd) { set_status(ERR_INVALID, "index_select: rank above 8 or bad dim"); return; }
    for (size_t d = 0; d < nd; ++d) out_dims[d] = d == dim ? n_idx : in_layout[d];
    IdxSpace sp; size_t n; Lay in;
    if (!make_space(nd, out_dims, dim, -1, sp, &n, "index_select: bad shape")) return;
    read_layout(nd, in_layout, in);
    if (n == 0) return;
    {
        constexpr int VEC = 16 / sizeof(T);
        size_t inner = 1;
        for (size_t d = dim + 1; d < nd; ++d) inner *= in_layout[d];
        const T* base = input + in_layout[2 * nd];
        if (ref_is_contiguous(nd, in_layout, in_layout + nd) && inner % VEC == 0 && ((uintptr_t)base % 16) == 0 && ((uintptr_t)output % 16) == 0 &&
            n_idx < (1ull << 31) && inner / VEC < (1ull << 31)) {
            size_t nvec = n / VEC;
            hipLaunchKernelGGL((index_select_rows_kernel<T, I, VEC>), dim3(cdiv(nvec, IB)), dim3(IB), 0, stream(), indices, (int64_t)idx_stride,
                               (int64_t)idx_offset, (uint32_t)n_idx, (uint32_t)in_layout[dim], (uint32_t)(inner / VEC),
                               make_fastdiv((uint32_t)(inner / VEC)), make_fastdiv((uint32_t)n_idx), base, output, nvec, flag);
            MXH_LAUNCH_CHECK("index_select");
            return;
        }
    }
    hipLaunchKernelGGL((index_select_kernel<T, I>), dim3(cdiv(n, IB)), dim3(IB), 0, stream(), sp, in, indices, (int64_t)idx_stride,
                       (int64_t)idx_offset, (uint32_t)in_layout[dim], input, output, n, flag);
    MXH_LAUNCH_CHECK("index_select");
}

template <class T, class I>
void gather(size_t nd, size_t dim, const size_t* in_layout, const size_t* idx_layout, const I* index, const T* input, T* output) {
    if (!in_layout || !idx_layout || !index || !input || !output) { set_status(ERR_INVALID, "gather: null argument"); return; }
    int* flag = index_flag();
    if (!flag) return;
    IdxSpace sp; size_t n; Lay in, ix;
    if (!make_space(nd, idx_layout, dim, -1, sp, &n, "gather: bad shape, rank above 8 or bad dim")) return;
    // the index tensor has the input's extent in every dim but `dim` (crates/maidenx_tensor/src/ops/indexing.rs:331-340):
    // a larger one would send the kernel past the end of the input
    for (size_t d = 0; d < nd; ++d)
        if (d != dim && idx_layout[d] != in_layout[d]) { set_status(ERR_INVALID, "gather: index and input shapes differ outside dim"); return; }
    read_layout(nd, in_layout, in);
    read_layout(nd, idx_layout, ix);
    if (n == 0) return;
    hipLaunchKernelGGL((gather_kernel<T, I>), dim3(cdiv(n, IB)), dim3(IB), 0, stream(), sp, in, ix, (uint32_t)in_layout[dim], index, input,
                       output, n, flag);
    MXH_LAUNCH_CHECK("gather");
}

template <class T, class I>
void index_add(size_t nd, size_t dim, const size_t* self_layout, const size_t* src_layout, size_t n_idx, size_t idx_stride,
               size_t idx_offset, const I* indices, const T* src, T* self) {
    if (!self_layout || !src_layout || !indices || !src || !self) { set_status(ERR_INVALID, "index_add_: null argument"); return; }
    int* flag = index_flag();
    if (!flag) return;
    IdxSpace sp; size_t lines; Lay sl, sr;
    if (!make_space(nd, self_layout, dim, (int)dim, sp, &lines, "index_add_: bad shape, rank above 8 or bad dim")) return;
    for (size_t d = 0; d < nd; ++d)
        if (d != dim && src_layout[d] != self_layout[d]) { set_status(ERR_INVALID, "index_add_: source and self differ outside dim"); return; }
    if (src_layout[dim] != n_idx) { set_status(ERR_INVALID, "index_add_: source extent along dim must equal the number of indices"); return; }
    if (n_idx >= (1ull << 31)) { set_status(ERR_TOO_LARGE, "index_add_: 2^31 or more indices"); return; }
    read_layout(nd, self_layout, sl);
    read_layout(nd, src_layout, sr);
    if (lines == 0 || n_idx == 0) return;
    const size_t D = self_layout[dim];
    if (n_idx >= 256 && lines < (1ull << 31) && D * lines < (1ull << 31) && D < (1ull << 31) - 1) {
        // [keys a | keys b | values a | values b | the sort's counts] in scratch slot 1
        unsigned bits = 1;
        while ((1ull << bits) <= D) ++bits;
        const size_t arr = (n_idx * sizeof(uint32_t) + 255) / 256 * 256;
        char* ws = (char*)scratch(4 * arr + rs_workspace_bytes(n_idx), 1);
        if (!ws) return;
        uint32_t *k_a = (uint32_t*)ws, *k_b = (uint32_t*)(ws + arr), *v_a = (uint32_t*)(ws + 2 * arr), *v_b = (uint32_t*)(ws + 3 * arr);
        hipLaunchKernelGGL(index_keys_kernel<I>, dim3(cdiv(n_idx, IB)), dim3(IB), 0, stream(), indices, (int64_t)idx_stride, (int64_t)idx_offset,
                           (uint32_t)n_idx, (uint32_t)D, k_a, v_a, flag);
        MXH_LAUNCH_CHECK("index_keys");
        prog_launch_seen();      // the sort's own launches
        const bool in_b = radix_sort_pairs_u32(k_a, v_a, k_b, v_b, n_idx, bits, (uint32_t*)(ws + 4 * arr), stream());
        MXH_LAUNCH_CHECK("radix_sort");
        const uint32_t *k_out = in_b ? k_b : k_a, *v_out = in_b ? v_b : v_a;
        {
            constexpr int VEC = 16 / sizeof(T);
            size_t inner = 1, outer = 1;
            for (size_t d = dim + 1; d < nd; ++d) inner *= self_layout[d];
            for (size_t d = 0; d < dim; ++d) outer *= self_layout[d];
            T* dbase = self + self_layout[2 * nd];
            const T* sbase = src + src_layout[2 * nd];
            const size_t inner_v = inner / VEC, chunks = cdiv(inner_v, (size_t)IB);
            if (ref_is_contiguous(nd, self_layout, self_layout + nd) && ref_is_contiguous(nd, src_layout, src_layout + nd) && inner % VEC == 0 &&
                ((uintptr_t)dbase % 16) == 0 && ((uintptr_t)sbase % 16) == 0 && outer * D * chunks < (1ull << 31)) {
                hipLaunchKernelGGL((index_add_rows_kernel<T, VEC>), dim3((unsigned)(outer * D * chunks)), dim3(IB), 0, stream(), k_out, v_out,
                                   (uint32_t)n_idx, (uint32_t)D, (uint32_t)inner_v, (uint32_t)chunks, make_fastdiv((uint32_t)chunks),
                                   make_fastdiv((uint32_t)D), sbase, dbase);
                MXH_LAUNCH_CHECK("index_add_rows");
                return;
            }
        }
        const size_t work = D * lines;
        hipLaunchKernelGGL(index_add_sorted_kernel<T>, dim3(cdiv(work, IB)), dim3(IB), 0, stream(), sp, sl, sr, k_out, v_out, (uint32_t)n_idx,
                           (uint32_t)lines, make_fastdiv((uint32_t)lines), src, self, work);
        MXH_LAUNCH_CHECK("index_add_sorted");
        return;
    }
    hipLaunchKernelGGL((index_add_kernel<T, I>), dim3(cdiv(lines, IB)), dim3(IB), 0, stream(), sp, sl, sr, indices, (int64_t)idx_stride,
                       (int64_t)idx_offset, (uint32_t)n_idx, (uint32_t)self_layout[dim], src, self, lines, flag);
    MXH_LAUNCH_CHECK("index_add");
}

template <class T, class I>
void scatter_add(size_t nd, size_t dim, const size_t* self_layout, const size_t* idx_layout, const size_t* src_layout, const I* index,
                 const T* src, T* self) {
    if (!self_layout || !idx_layout || !src_layout || !index || !src || !self) { set_status(ERR_INVALID, "scatter_add_: null argument"); return; }
    int* flag = index_flag();
    if (!flag) return;
    IdxSpace sp; size_t lines; Lay sl, ix, sr;
    if (!make_space(nd, src_layout, dim, (int)dim, sp, &lines, "scatter_add_: bad shape, rank above 8 or bad dim")) return;
    for (size_t d = 0; d < nd; ++d) {
        if (src_layout[d] != idx_layout[d]) { set_status(ERR_INVALID, "scatter_add_: source and index shapes differ"); return; }
        // add_at_index (utils/indexing.rs:105-112) refuses coordinates beyond self
        if (d != dim && src_layout[d] > self_layout[d]) { set_status(ERR_INVALID, "scatter_add_: source exceeds self outside dim"); return; }
    }
    if (src_layout[dim] >= (1ull << 31) || self_layout[dim] >= (1ull << 31)) { set_status(ERR_TOO_LARGE, "scatter_add_: dim of 2^31 or more"); return; }
    read_layout(nd, self_layout, sl);
    read_layout(nd, idx_layout, ix);
    read_layout(nd, src_layout, sr);
    if (lines == 0 || src_layout[dim] == 0) return;
    hipLaunchKernelGGL((scatter_add_kernel<T, I>), dim3(cdiv(lines, IB)), dim3(IB), 0, stream(), sp, sl, ix, sr, (uint32_t)src_layout[dim],
                       (uint32_t)self_layout[dim], index, src, self, lines, flag);
    MXH_LAUNCH_CHECK("scatter_add");
}

template <class I>
void bincount(size_t n, size_t stride, size_t offset, const I* input, size_t out_size, I* output) {
    if (!input || !output) { set_status(ERR_INVALID, "bincount: null argument"); return; }
    int* flag = index_flag();
    if (!flag) return;
    if (n >= (1ull << 40) || out_size >= (1ull << 31)) { set_status(ERR_TOO_LARGE, "bincount: too large"); return; }
    if (out_size == 0) return;
    hipLaunchKernelGGL(zero_counts_kernel<I>, dim3(cdiv(out_size, IB)), dim3(IB), 0, stream(), output, out_size);
    if (n) hipLaunchKernelGGL(bincount_kernel<I>, dim3(cdiv(n, IB)), dim3(IB), 0, stream(), input, (int64_t)stride, (int64_t)offset, n, output, out_size, flag);
    MXH_LAUNCH_CHECK("bincount");
}

template <class T, class I>
void bincount_weighted(size_t n, size_t stride, size_t offset, const I* input, size_t w_stride, size_t w_offset, const T* weights,
                       size_t out_size, T* output) {
    if (!input || !weights || !output) { set_status(ERR_INVALID, "bincount: null argument"); return; }
    int* flag = index_flag();
    if (!flag) return;
    // every bin's thread scans the whole input: fine for the label-count sizes this is used at
    if (out_size >= (1ull << 31) || (double)n * (double)out_size > 1.0e12) { set_status(ERR_TOO_LARGE, "bincount with weights: input x bins above 1e12"); return; }
    if (out_size == 0) return;
    hipLaunchKernelGGL((bincount_weighted_kernel<T, I>), dim3(cdiv(out_size, IB)), dim3(IB), 0, stream(), input, (int64_t)stride,
                       (int64_t)offset, weights, (int64_t)w_stride, (int64_t)w_offset, n, output, out_size, flag);
    MXH_LAUNCH_CHECK("bincount_weighted");
}

// ---- index_put_ (tensor/ops/indexing.rs:182-311) ---------------------------------------------------------
// `indices` fixes the leading dims of self; src (whose shape must equal self's remaining dims) is copied into that
// sub-tensor through the strides of both.  With every dim fixed, a 0-d src is one element written at that
// position, and any other src is written element by element (read with its stride 0 only, as the reference does)
// to positions indices[0], indices[0] + 1, ... of a 1-d self.  The copy is the in-place elementwise path with an
// "assign" functor.  Positions of self that alias each other (stride 0) are written in no particular order.
template <class T>
void index_put(size_t self_nd, const size_t* self_layout, size_t n_indices, const size_t* indices, size_t src_nd,
               const size_t* src_layout, const T* src, T* self) {
    if (!self_layout || !src_layout || !src || !self || (n_indices && !indices)) { set_status(ERR_INVALID, "index_put_: null argument"); return; }
    if (self_nd > 64 || src_nd > 64) { set_status(ERR_INVALID, "index_put_: rank above 64"); return; }
    if (n_indices > self_nd) { set_status(ERR_INVALID, "index_put_: more indices than dims"); return; }
    const size_t *sd = self_layout, *ss = self_layout + self_nd, *rd = src_layout, *rs = src_layout + src_nd;
    const size_t self_off = self_layout[2 * self_nd], src_off = src_layout[2 * src_nd];
    const size_t remaining = self_nd - n_indices;
    size_t md[3 * 64 + 2];
    size_t nd = 0, num_els = 1, base = self_off;
    if (remaining > 0) {
        if (src_nd != remaining) { set_status(ERR_INVALID, "index_put_: source rank differs from the remaining dims"); return; }
        for (size_t i = 0; i < remaining; ++i)
            if (rd[i] != sd[n_indices + i]) { set_status(ERR_INVALID, "index_put_: source shape differs from the remaining dims"); return; }
        for (size_t d = 0; d < n_indices; ++d) {
            if (indices[d] >= sd[d]) { set_status(ERR_INVALID, "index_put_: index out of bounds"); return; }
            base += indices[d] * ss[d];
        }
        nd = remaining;
        for (size_t i = 0; i < nd; ++i) { md[i] = rd[i]; md[nd + i] = ss[n_indices + i]; md[2 * nd + i] = rs[i]; num_els *= rd[i]; }
    } else if (src_nd == 0) {
        for (size_t d = 0; d < n_indices; ++d) {
            if (indices[d] >= sd[d]) { set_status(ERR_INVALID, "index_put_: index out of bounds"); return; }
            base += indices[d] * ss[d];
        }
        nd = 1; md[0] = 1; md[1] = 1; md[2] = 1;
    } else {
        size_t src_size = 1, self_size = 1;
        for (size_t i = 0; i < src_nd; ++i) src_size *= rd[i];
        for (size_t i = 0; i < self_nd; ++i) self_size *= sd[i];
        if (src_size == 0) return;
        if (self_nd == 0) { set_status(ERR_INVALID, "index_put_: no index for a non-scalar source"); return; }
        if (indices[0] + src_size > self_size) { set_status(ERR_INVALID, "index_put_: source does not fit behind the index"); return; }
        if (self_nd != 1) { set_status(ERR_INVALID, "index_put_: a flat copy needs a 1-d destination"); return; }
        base += indices[0] * ss[0];
        nd = 1; md[0] = src_size; md[1] = ss[0]; md[2] = rs[0]; num_els = src_size;
    }
    if (num_els == 0) return;
    md[3 * nd] = base;
    md[3 * nd + 1] = src_off;
    ew_binary(num_els, nd, md, self, src, nullptr, OpAssign<T>{}, true);
}

}  // namespace mxh

using namespace mxh;

#define MXH_INDEX_PUT_FOR(T, TS)                                                                                                    \
    extern "C" void hip_index_put_##TS(size_t self_nd, const size_t* self_layout, size_t n_indices, const size_t* indices,          \
                                       size_t src_nd, const size_t* src_layout, const T* src, T* self) { MXH_API;                   \
        index_put<T>(self_nd, self_layout, n_indices, indices, src_nd, src_layout, src, self);                                      \
    }
MXH_INDEX_PUT_FOR(float, f32)
MXH_INDEX_PUT_FOR(bf16_t, bf16)
MXH_INDEX_PUT_FOR(f16_t, f16)

#define MXH_INDEX_FOR(T, TS, I, IS)                                                                                                  \
    extern "C" void hip_index_select_##TS##_##IS(size_t nd, size_t dim, const size_t* in_layout, size_t n_idx, size_t idx_stride,    \
                                                 size_t idx_offset, const I* indices, const T* input, T* output) { MXH_API;          \
        index_select<T, I>(nd, dim, in_layout, n_idx, idx_stride, idx_offset, indices, input, output);                               \
    }                                                                                                                                \
    extern "C" void hip_gather_##TS##_##IS(size_t nd, size_t dim, const size_t* in_layout, const size_t* idx_layout, const I* index, \
                                           const T* input, T* output) { MXH_API;                                                    \
        gather<T, I>(nd, dim, in_layout, idx_layout, index, input, output);                                                          \
    }                                                                                                                                \
    extern "C" void hip_index_add_##TS##_##IS(size_t nd, size_t dim, const size_t* self_layout, const size_t* src_layout,            \
                                              size_t n_idx, size_t idx_stride, size_t idx_offset, const I* indices, const T* src,   \
                                              T* self) { MXH_API;                                                                    \
        index_add<T, I>(nd, dim, self_layout, src_layout, n_idx, idx_stride, idx_offset, indices, src, self);                        \
    }                                                                                                                                \
    extern "C" void hip_scatter_add_##TS##_##IS(size_t nd, size_t dim, const size_t* self_layout, const size_t* idx_layout,          \
                                                const size_t* src_layout, const I* index, const T* src, T* self) { MXH_API;         \
        scatter_add<T, I>(nd, dim, self_layout, idx_layout, src_layout, index, src, self);                                           \
    }                                                                                                                                \
    extern "C" void hip_bincount_weighted_##TS##_##IS(size_t n, size_t stride, size_t offset, const I* input, size_t w_stride,       \
                                                      size_t w_offset, const T* weights, size_t out_size, T* output) { MXH_API;     \
        bincount_weighted<T, I>(n, stride, offset, input, w_stride, w_offset, weights, out_size, output);                            \
    }

// f64, bool and the integers: the tensor layer's index ops are dtype-generic (indexing.rs:15, 93, 182, 315, 403 go through
// Scalar), so every storage dtype has them; the weighted bincount is for float weights (f64 here besides the three above)
#define MXH_INDEX_WIDE_FOR(T, P, TS, I, IS)                                                                                          \
    extern "C" void hip_index_select_##TS##_##IS(size_t nd, size_t dim, const size_t* in_layout, size_t n_idx, size_t idx_stride,    \
                                                 size_t idx_offset, const I* indices, const P* input, P* output) { MXH_API;          \
        index_select<T, I>(nd, dim, in_layout, n_idx, idx_stride, idx_offset, indices, (const T*)input, (T*)output);                 \
    }                                                                                                                                \
    extern "C" void hip_gather_##TS##_##IS(size_t nd, size_t dim, const size_t* in_layout, const size_t* idx_layout, const I* index, \
                                           const P* input, P* output) { MXH_API;                                                    \
        gather<T, I>(nd, dim, in_layout, idx_layout, index, (const T*)input, (T*)output);                                            \
    }                                                                                                                                \
    extern "C" void hip_index_add_##TS##_##IS(size_t nd, size_t dim, const size_t* self_layout, const size_t* src_layout,            \
                                              size_t n_idx, size_t idx_stride, size_t idx_offset, const I* indices, const P* src,   \
                                              P* self) { MXH_API;                                                                    \
        index_add<T, I>(nd, dim, self_layout, src_layout, n_idx, idx_stride, idx_offset, indices, (const T*)src, (T*)self);          \
    }                                                                                                                                \
    extern "C" void hip_scatter_add_##TS##_##IS(size_t nd, size_t dim, const size_t* self_layout, const size_t* idx_layout,          \
                                                const size_t* src_layout, const I* index, const P* src, P* self) { MXH_API;         \
        scatter_add<T, I>(nd, dim, self_layout, idx_layout, src_layout, index, (const T*)src, (T*)self);                             \
    }
#define MXH_INDEX_WIDE(T, P, TS)                                                                                                     \
    MXH_INDEX_WIDE_FOR(T, P, TS, int32_t, i32) MXH_INDEX_WIDE_FOR(T, P, TS, int64_t, i64)                                            \
    extern "C" void hip_index_put_##TS(size_t self_nd, const size_t* self_layout, size_t n_indices, const size_t* indices,          \
                                       size_t src_nd, const size_t* src_layout, const P* src, P* self) { MXH_API;                   \
        index_put<T>(self_nd, self_layout, n_indices, indices, src_nd, src_layout, (const T*)src, (T*)self);                        \
    }
MXH_INDEX_WIDE(double, double, f64)
MXH_INDEX_WIDE(b8_t, uint8_t, bool)
MXH_INDEX_WIDE(uint8_t, uint8_t, u8)
MXH_INDEX_WIDE(uint16_t, uint16_t, u16)
MXH_INDEX_WIDE(uint32_t, uint32_t, u32)
MXH_INDEX_WIDE(uint64_t, uint64_t, u64)
MXH_INDEX_WIDE(int8_t, int8_t, i8)
MXH_INDEX_WIDE(int16_t, int16_t, i16)
MXH_INDEX_WIDE(int32_t, int32_t, i32)
MXH_INDEX_WIDE(int64_t, int64_t, i64)
extern "C" void hip_bincount_weighted_f64_i32(size_t n, size_t stride, size_t offset, const int32_t* input, size_t w_stride, size_t w_offset,
                                              const double* weights, size_t out_size, double* output) { MXH_API;
    bincount_weighted<double, int32_t>(n, stride, offset, input, w_stride, w_offset, weights, out_size, output);
}
extern "C" void hip_bincount_weighted_f64_i64(size_t n, size_t stride, size_t offset, const int64_t* input, size_t w_stride, size_t w_offset,
                                              const double* weights, size_t out_size, double* output) { MXH_API;
    bincount_weighted<double, int64_t>(n, stride, offset, input, w_stride, w_offset, weights, out_size, output);
}

MXH_INDEX_FOR(float, f32, int32_t, i32)
MXH_INDEX_FOR(float, f32, int64_t, i64)
MXH_INDEX_FOR(bf16_t, bf16, int32_t, i32)
MXH_INDEX_FOR(bf16_t, bf16, int64_t, i64)
MXH_INDEX_FOR(f16_t, f16, int32_t, i32)
MXH_INDEX_FOR(f16_t, f16, int64_t, i64)

extern "C" void hip_bincount_i32(size_t n, size_t stride, size_t offset, const int32_t* input, size_t out_size, int32_t* output) { MXH_API;
    bincount<int32_t>(n, stride, offset, input, out_size, output);
}
extern "C" void hip_bincount_i64(size_t n, size_t stride, size_t offset, const int64_t* input, size_t out_size, int64_t* output) { MXH_API;
    bincount<int64_t>(n, stride, offset, input, out_size, output);
}
