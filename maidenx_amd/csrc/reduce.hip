// Reductions: sum / mean / max / min along one axis and sum_to_shape.  They replace the
// `cuda_<op>_<dtype>` symbols of crates/maidenx_cuda/src/ops/reduction.rs:19-35 and follow the
// CPU semantics of crates/maidenx_cpu/src/ops/reduction.rs.
//
// A contiguous input reduced along one axis is the 3-d problem [outer, L, S] → [outer, S]:
//   S == 1 : "row" reduce.  One thread, one wave or one block per row (by row length); lanes
//            read 128-bit vectors, partial sums meet in a wave64 DPP butterfly and then in LDS.
//   S  > 1 : "column" reduce.  Lanes run along S (coalesced, 128-bit where alignment allows)
//            and walk L; when outer*S alone cannot fill the chip, L is cut into chunks whose
//            partial results go to library scratch and are folded by a second launch.  Wide rows
//            with a long axis use blocks of 16 waves that share 64 column vectors and split the
//            axis among the waves (partials meet in LDS), so fewer chunks are needed.
// sum_to_shape folds its reduced groups with these two, innermost first; the [reduced, kept, reduced]
// shape of a per-channel gradient has a one-pass kernel of its own.
// Accumulation is f32 in a fixed order (deterministic from run to run); bf16 is rounded once.
// No atomics anywhere.
#include <cfloat>
#include <mutex>

#include "elementwise.hpp"
#include "mxh.hpp"
#include "ops.hpp"
#include "reduce_row.hpp"

namespace mxh {

constexpr size_t COL_SPLIT_BLOCKS = 256;      // one 16-wave block per CU

// ---- where the chunk partials live ---------------------------------------------------------------------
// Normally in the library's scratch slot 0, which is allocated and grown on demand.  The entry points that must not
// allocate (hip_sum_f32_noalloc) keep them in a fixed array that is part of the code object instead: every device the
// library runs on holds its own copy of it from the first use of the library to the end of the process.
constexpr size_t FIXED_PARTIALS_BYTES = 4u << 20;
static __device__ __align__(256) unsigned char g_fixed_partials[FIXED_PARTIALS_BYTES];
static std::mutex g_fixed_mu;
static void* g_fixed_ptr[16] = {nullptr};            // device address of the array, per device (the name above is a host-side stand-in)
static thread_local void* t_fixed = nullptr;         // set while a no-alloc entry point runs on this thread

// Device address of this device's copy of the array; resolved once per device, with that device current.
static void* fixed_partials() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) { set_status(ERR_INVALID, "no-alloc reduce: bad device"); return nullptr; }
    std::lock_guard<std::mutex> lk(g_fixed_mu);
    if (!g_fixed_ptr[dev]) {
        void* p = nullptr;
        hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(g_fixed_partials));
        if (e != hipSuccess || !p) { set_status(ERR_LAUNCH, "no-alloc reduce: hipGetSymbolAddress", (int)e); return nullptr; }
        g_fixed_ptr[dev] = p;
    }
    return g_fixed_ptr[dev];
}

// The array is cut in two: chunk partials in the first 3 MiB, the partial rows of a regrouped narrow-row reduction
// (col_reduce below) in the last one.
constexpr size_t FIXED_CHUNK_BYTES = 3u << 20;
constexpr size_t FIXED_REGROUP_BYTES = FIXED_PARTIALS_BYTES - FIXED_CHUNK_BYTES;

static float* partials(size_t bytes) {
    if (!t_fixed) return (float*)scratch(bytes);
    if (bytes > FIXED_CHUNK_BYTES) {
        set_status(ERR_TOO_LARGE, "no-alloc reduce: the chunk partials of this shape exceed their 3 MiB of the fixed array; use the allocating entry point");
        return nullptr;
    }
    return (float*)t_fixed;
}

// Partial rows of a regrouped reduction: scratch slot 2, or the last MiB of the fixed array.
static float* regroup_rows(size_t bytes) {
    if (!t_fixed) return (float*)scratch(bytes, 2);
    if (bytes > FIXED_REGROUP_BYTES) {
        set_status(ERR_TOO_LARGE, "no-alloc reduce: the regrouped partial rows of this shape exceed their 1 MiB of the fixed array; use the allocating entry point");
        return nullptr;
    }
    return (float*)((unsigned char*)t_fixed + FIXED_CHUNK_BYTES);
}

// ---- column reduce: [outer, L, S] → [outer, chunks, S] ------------------------------------------
template <class TIn, class TOut, class R, int VEC, bool STREAM = false>
__global__ __launch_bounds__(RB) void col_reduce_kernel(const TIn* __restrict__ in, TOut* __restrict__ out, size_t outer,
                                                        size_t L, size_t S, unsigned chunks, size_t chunk_len,
                                                        FastDiv div_sv, FastDiv div_chunks, size_t total, float div,
                                                        bool src_bf16) {
    size_t tid = (size_t)blockIdx.x * RB + threadIdx.x;
    if (tid >= total) return;
    // tid → (o, chunk, jv), jv fastest.  total < 2^32 is checked by the host.
    uint32_t rest, jv, o, chunk;
    fd_divmod((uint32_t)tid, div_sv, rest, jv);
    fd_divmod(rest, div_chunks, o, chunk);
    size_t beg = (size_t)chunk * chunk_len, end = beg + chunk_len < L ? beg + chunk_len : L;
    const TIn* src = in + ((size_t)o * L + beg) * S + (size_t)jv * VEC;
    float a[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) a[e] = R::init(src_bf16);
#pragma unroll 8
    for (size_t l = beg; l < end; ++l, src += S) {
        AVec<TIn, VEC> v = ld_vec<STREAM>((const AVec<TIn, VEC>*)src);
#pragma unroll
        for (int e = 0; e < VEC; ++e) a[e] = R::op(a[e], IO<TIn>::ld(v.v[e]));
    }
    AVec<TOut, VEC> r;
#pragma unroll
    for (int e = 0; e < VEC; ++e) r.v[e] = IO<TOut>::fin(a[e], div);
    *(AVec<TOut, VEC>*)(out + ((size_t)o * chunks + chunk) * S + (size_t)jv * VEC) = r;
}

// ---- column reduce with the reduced axis split inside the block -------------------------------------
// A block is NW waves deep: wave w walks slice w of the chunk's rows for
// the same 64 column vectors, COL_U loads in flight per lane, and the NW partial rows meet in LDS in wave
// order.  Against one thread per column this multiplies the loads in flight without more partials to
// write and fold.  Requires S % VEC == 0 and aligned bases.
template <class TIn, class TOut, class R, int VEC, int NW, bool STREAM = false>
__global__ __launch_bounds__(WAVE * NW) void col_reduce_split_kernel(const TIn* __restrict__ in, TOut* __restrict__ out, size_t L,
                                                                      size_t S, uint32_t sv, unsigned chunks, size_t chunk_len,
                                                                      FastDiv div_jb, FastDiv div_chunks, float div, bool src_bf16) {
    constexpr int U = 8;
    const int lane = threadIdx.x % WAVE, w = threadIdx.x / WAVE;
    uint32_t rest, jb, o, chunk;
    fd_divmod(blockIdx.x, div_jb, rest, jb);
    fd_divmod(rest, div_chunks, o, chunk);
    const uint32_t jv = jb * WAVE + lane;
    const bool live = jv < sv;
    const size_t beg = (size_t)chunk * chunk_len, end = beg + chunk_len < L ? beg + chunk_len : L;
    const size_t slice = (end - beg + NW - 1) / NW;
    const size_t l0 = beg + (size_t)w * slice < end ? beg + (size_t)w * slice : end, l1 = l0 + slice < end ? l0 + slice : end;
    float a[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) a[e] = R::init(src_bf16);
    if (live) {
        const TIn* src = in + ((size_t)o * L + l0) * S + (size_t)jv * VEC;
        size_t l = l0;
        for (; l + U <= l1; l += U, src += U * S) {
            AVec<TIn, VEC> v[U];
#pragma unroll
            for (int k = 0; k < U; ++k) v[k] = ld_vec<STREAM>((const AVec<TIn, VEC>*)(src + k * S));
#pragma unroll
            for (int k = 0; k < U; ++k)
#pragma unroll
                for (int e = 0; e < VEC; ++e) a[e] = R::op(a[e], IO<TIn>::ld(v[k].v[e]));
        }
        for (; l < l1; ++l, src += S) {
            AVec<TIn, VEC> v = *(const AVec<TIn, VEC>*)src;
#pragma unroll
            for (int e = 0; e < VEC; ++e) a[e] = R::op(a[e], IO<TIn>::ld(v.v[e]));
        }
    }
    __shared__ float part[NW][VEC][WAVE];
#pragma unroll
    for (int e = 0; e < VEC; ++e) part[w][e][lane] = a[e];
    __syncthreads();
    if (w == 0 && live) {
        AVec<TOut, VEC> r;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            float t = part[0][e][lane];
#pragma unroll
            for (int k = 1; k < NW; ++k) t = R::op(t, part[k][e][lane]);
            r.v[e] = IO<TOut>::fin(t, div);
        }
        *(AVec<TOut, VEC>*)(out + ((size_t)o * chunks + chunk) * S + (size_t)jv * VEC) = r;
    }
}

// ---- plane reduce: [A, K, S] → [chunks, K], summing over a and s ------------------------------------
// The gradient of a per-channel parameter ([B, C, H*W] → [1, C, 1]): every kept index k owns A
// separate runs of S contiguous elements.  One block of PB threads per (k, chunk of rows a); the
// threads sweep the runs as 16-byte vectors, four loads in flight each, then meet in a DPP
// butterfly and LDS.  S % VEC == 0 and a 16-byte aligned base are required.
constexpr int PLB = 1024;
template <class TIn, class TOut, class R, int VEC, bool STREAM = false>
__global__ __launch_bounds__(PLB) void plane_reduce_kernel(const TIn* __restrict__ in, TOut* __restrict__ out, uint32_t A,
                                                           uint32_t K, uint32_t S, uint32_t a_chunk, FastDiv div_sv,
                                                           bool src_bf16) {
    const uint32_t k = blockIdx.x % K, chunk = blockIdx.x / K;
    const uint32_t a0 = chunk * a_chunk, rows = min(a_chunk, A - a0);
    const uint32_t sv = S / VEC, nvec = rows * sv;
    const TIn* base = in + ((size_t)a0 * K + k) * S;
    const size_t row_pitch = (size_t)K * S;
    float acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] = R::init(src_bf16);
    auto addr = [&](uint32_t f) {
        uint32_t a, c;
        fd_divmod(f, div_sv, a, c);
        return base + a * row_pitch + (size_t)c * VEC;
    };
    uint32_t f = threadIdx.x;
    for (; f + 3 * PLB < nvec; f += 4 * PLB) {
        AVec<TIn, VEC> v[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) v[q] = ld_vec<STREAM>((const AVec<TIn, VEC>*)addr(f + q * PLB));
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int e = 0; e < VEC; ++e) acc[e] = R::op(acc[e], IO<TIn>::ld(v[q].v[e]));
    }
    for (; f < nvec; f += PLB) {
        AVec<TIn, VEC> v = *(const AVec<TIn, VEC>*)addr(f);
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] = R::op(acc[e], IO<TIn>::ld(v.v[e]));
    }
    float r = acc[0];
#pragma unroll
    for (int e = 1; e < VEC; ++e) r = R::op(r, acc[e]);
    r = wave_reduce<R>(r);
    __shared__ float part[PLB / WAVE];
    if (threadIdx.x % WAVE == 0) part[threadIdx.x / WAVE] = r;
    __syncthreads();
    if (threadIdx.x == 0) {
        r = part[0];
#pragma unroll
        for (int w = 1; w < PLB / WAVE; ++w) r = R::op(r, part[w]);
        out[(size_t)chunk * K + k] = IO<TOut>::fin(r, 0.0f);
    }
}

// ---- generic single-axis reduce over a strided input (the reference's non-contiguous branch) ----
// One thread per output element d; its inputs are the logical indices ((d/s)*L + l)*s + d%s
// (s = the metadata's reduced stride, or d*L + l when that stride is 0), each mapped through the
// strides the way get_strided_index does.
template <class T, class R>
__global__ __launch_bounds__(RB) void reduce_generic_kernel(NdSpace<1> sp, const T* __restrict__ in, T* __restrict__ out,
                                                            size_t num_els, size_t out_size, size_t L, size_t s,
                                                            float div) {
    size_t d = (size_t)blockIdx.x * RB + threadIdx.x;
    if (d >= out_size) return;
    float acc = R::init(IO<T>::is_bf16);
    for (size_t l = 0; l < L; ++l) {
        size_t i = s != 0 ? ((d / s) * L + l) * s + d % s : d * L + l;
        if (i >= num_els) continue;
        uint32_t r = (uint32_t)i;
        int64_t off = 0;
        for (int k = sp.ndims - 1; k > 0; --k) {
            uint32_t q, c;
            fd_divmod(r, sp.div[k], q, c);
            off += (int64_t)c * sp.strides[0][k];
            r = q;
        }
        off += (int64_t)r * sp.strides[0][0];
        acc = R::op(acc, IO<T>::ld(in[off]));
    }
    out[d] = IO<T>::fin(acc, div);
}

// ---- host drivers ---------------------------------------------------------------------------------
constexpr size_t TARGET_BLOCKS = 2048;   // 256 CUs x 8 resident blocks
// Column reductions keep 8 independent 16-byte loads in flight per thread, so two blocks per CU already cover the
// memory latency; longer chunks mean fewer partials to write and fold (measured best on [8192,8192] and [64,512,1024]).
constexpr size_t COL_TARGET_BLOCKS = 512;
constexpr size_t COL_MIN_ROWS = 128;

template <class T> inline bool aligned16(const T* p) { return ((uintptr_t)p & 15u) == 0; }

// An input of this many bytes is read once and cannot be in any cache when it is next needed: its loads then carry the
// non-temporal hint (a read-only sweep of 268 MB: 44 -> 40 us).  Same threshold as the elementwise kernels.
inline bool streams(size_t input_bytes) { return ew_stream_bytes() != 0 && input_bytes >= ew_stream_bytes() / 2; }

template <class TIn, class TOut, class R, int TPR>
void launch_row(const TIn* in, TOut* out, size_t rows, size_t L, unsigned chunks, size_t chunk_len, float div,
                bool src_bf16) {
    constexpr int VEC = 16 / sizeof(TIn);
    constexpr int RPB = RB / TPR;
    unsigned blocks = cdiv(rows * chunks, RPB);
    bool vec = aligned16(in) && L % VEC == 0 && chunk_len % VEC == 0;
    if constexpr (std::is_same<TIn, float>::value && std::is_same<TOut, float>::value) {
        RowProgArgs a;
        std::memset((void*)&a, 0, sizeof(a));
        a.in = in; a.out = out; a.rows = rows; a.L = L; a.chunks = chunks; a.chunk_len = chunk_len; a.div = div; a.src_bf16 = src_bf16;
        const bool small = blocks <= PROG_MAX_GRID && rows * L <= PROG_MAX_ELEMS;
        if (prog_recording() && !small) prog_abandon();
        if constexpr (std::is_same<R, RSum>::value) {
            // a sum that one work-group does anyway: a stage in the tail of the open chain of fused launches
            static_assert(sizeof(RowProgArgs) <= FUSE_TAIL_ARG_BYTES, "a tail stage holds a row reduction's arguments");
            if (capture_open() && blocks == 1 && rows * L <= 65536) {
                const Extent src{(uintptr_t)in, (uintptr_t)in + rows * L * sizeof(float)};
                const Extent dst{(uintptr_t)out, (uintptr_t)out + rows * chunks * sizeof(float)};
                if (fuse_record_tail(TAIL_ROW_REDUCE, row_prog_sub<R, TPR>(vec ? 1 : 0), &a, sizeof(a), &src, 1, dst, rows * chunks)) return;
            }
        }
        if (prog_recording() && small) prog_record(prog_kid(PF_ROW_REDUCE, row_prog_sub<R, TPR>(vec ? 1 : 0)), blocks, &a, sizeof(a));
    }
    if (vec && streams(rows * L * sizeof(TIn)))
        hipLaunchKernelGGL((row_reduce_kernel<TIn, TOut, R, TPR, VEC, true>), dim3(blocks), dim3(RB), 0, stream(), in, out, rows,
                           L, chunks, chunk_len, div, src_bf16);
    else if (vec)
        hipLaunchKernelGGL((row_reduce_kernel<TIn, TOut, R, TPR, VEC>), dim3(blocks), dim3(RB), 0, stream(), in, out, rows,
                           L, chunks, chunk_len, div, src_bf16);
    else
        hipLaunchKernelGGL((row_reduce_kernel<TIn, TOut, R, TPR, 1>), dim3(blocks), dim3(RB), 0, stream(), in, out, rows,
                           L, chunks, chunk_len, div, src_bf16);
    MXH_LAUNCH_CHECK("row_reduce");
}

template <class TIn, class TOut, class R>
void row_stage(const TIn* in, TOut* out, size_t rows, size_t L, unsigned chunks, size_t chunk_len, float div,
               bool src_bf16) {
    size_t len = chunks > 1 ? chunk_len : L;
    // many rows of a few dozen elements (the sums over the last dim of an image batch, rows of 56): a wave per row would
    // leave three lanes in four without an element; 16 lanes per row, four rows per wave
    constexpr int V16 = 16 / sizeof(TIn);
    if (len > 32 && len <= 64 * V16 && rows * chunks >= 65536 && aligned16(in) && L % V16 == 0 && chunk_len % V16 == 0) {
        if constexpr (std::is_same<TIn, float>::value && std::is_same<TOut, float>::value)
            if (prog_recording()) prog_abandon();          // (far beyond what a recorded program holds)
        const unsigned blocks = cdiv(rows * chunks, (size_t)(RB / 16));
        if (streams(rows * L * sizeof(TIn)))
            hipLaunchKernelGGL((row_reduce_kernel<TIn, TOut, R, 16, V16, true>), dim3(blocks), dim3(RB), 0, stream(), in, out, rows, L, chunks,
                               chunk_len, div, src_bf16);
        else
            hipLaunchKernelGGL((row_reduce_kernel<TIn, TOut, R, 16, V16>), dim3(blocks), dim3(RB), 0, stream(), in, out, rows, L, chunks,
                               chunk_len, div, src_bf16);
        MXH_LAUNCH_CHECK("row_reduce");
        return;
    }
    if (len <= 32) launch_row<TIn, TOut, R, 1>(in, out, rows, L, chunks, chunk_len, div, src_bf16);
    else if (len <= 2048) launch_row<TIn, TOut, R, WAVE>(in, out, rows, L, chunks, chunk_len, div, src_bf16);
    else launch_row<TIn, TOut, R, RB>(in, out, rows, L, chunks, chunk_len, div, src_bf16);
}

// `0 + x` per element: what an all-kept sum_to_shape does through its zero-initialised cells (−0 → +0), and what a
// sum over an axis of length 1 is.
template <class T> struct OpZeroPlus {
    using In = T; using Out = T; static constexpr int NIN = 1;
    __device__ T operator()(T x) const { return IO<T>::fin(0.0f + IO<T>::ld(x), 0.0f); }
};

// rows of length L (contiguous) → out[rows]
template <class TIn, class TOut, class R>
void row_reduce(const TIn* in, TOut* out, size_t rows, size_t L, float div, bool src_bf16) {
    if constexpr (std::is_same<TIn, TOut>::value && std::is_same<R, RSum>::value) {
        if (L == 1 && div == 0.0f) {
            // one term per row: the sum is `0 + x`, an elementwise launch (which a capture can fuse with its neighbours)
            size_t dims = rows, unit = 1;
            const size_t* ins[1] = {&unit};
            const void* inp[1] = {in};
            ew_launch<OpZeroPlus<TIn>>(rows, 1, &dims, &unit, ins, out, inp, OpZeroPlus<TIn>{});
            return;
        }
    }
    unsigned chunks = 1;
    size_t chunk_len = L;
    if (rows < TARGET_BLOCKS / 4 && L >= 16384) {
        size_t want = TARGET_BLOCKS / rows;
        size_t max_chunks = L / 4096;              // keep at least 4096 elements per chunk
        chunks = (unsigned)(want < max_chunks ? want : max_chunks);
        if (chunks < 1) chunks = 1;
        chunk_len = ((L + chunks - 1) / chunks + 63) / 64 * 64;
        chunks = (unsigned)((L + chunk_len - 1) / chunk_len);
    }
    if (chunks == 1) { row_stage<TIn, TOut, R>(in, out, rows, L, 1, L, div, src_bf16); return; }
    float* part = partials(rows * chunks * sizeof(float) + 256);
    if (!part) return;
    row_stage<TIn, float, R>(in, part, rows, L, chunks, chunk_len, 0.0f, src_bf16);
    row_stage<float, TOut, R>(part, out, rows, chunks, 1, chunks, div, src_bf16);
}

template <class TIn, class TOut, class R>
void col_stage(const TIn* in, TOut* out, size_t outer, size_t L, size_t S, unsigned chunks, size_t chunk_len, float div,
               bool src_bf16) {
    constexpr int VI = 16 / sizeof(TIn), VO = 16 / sizeof(TOut);
    constexpr int VEC = VI < VO ? VI : VO;
    bool vec = S % VEC == 0 && ((uintptr_t)in % (VEC * sizeof(TIn))) == 0 && ((uintptr_t)out % (VEC * sizeof(TOut))) == 0;
    size_t sv = vec ? S / VEC : S;
    size_t total = outer * chunks * sv;
    if (total >= (1ull << 32)) { set_status(ERR_TOO_LARGE, "column reduce: more than 2^32 work items"); return; }
    unsigned blocks = cdiv(total, RB);
    FastDiv dsv = make_fastdiv((uint32_t)sv), dch = make_fastdiv(chunks);
    if constexpr (VEC == 8) {
        // 16-bit elements and few threads (one wave per SIMD or less): 8-byte vectors double the waves, which
        // hides the unpacking arithmetic behind the loads
        if (vec && blocks <= 256) {
            size_t sv4 = S / 4, total4 = outer * chunks * sv4;
            hipLaunchKernelGGL((col_reduce_kernel<TIn, TOut, R, 4>), dim3(cdiv(total4, RB)), dim3(RB), 0, stream(), in, out, outer, L, S,
                               chunks, chunk_len, make_fastdiv((uint32_t)sv4), dch, total4, div, src_bf16);
            MXH_LAUNCH_CHECK("col_reduce");
            return;
        }
    }
    if (vec && streams(outer * L * S * sizeof(TIn)))
        hipLaunchKernelGGL((col_reduce_kernel<TIn, TOut, R, VEC, true>), dim3(blocks), dim3(RB), 0, stream(), in, out, outer, L, S,
                           chunks, chunk_len, dsv, dch, total, div, src_bf16);
    else if (vec)
        hipLaunchKernelGGL((col_reduce_kernel<TIn, TOut, R, VEC>), dim3(blocks), dim3(RB), 0, stream(), in, out, outer, L, S,
                           chunks, chunk_len, dsv, dch, total, div, src_bf16);
    else
        hipLaunchKernelGGL((col_reduce_kernel<TIn, TOut, R, 1>), dim3(blocks), dim3(RB), 0, stream(), in, out, outer, L, S,
                           chunks, chunk_len, dsv, dch, total, div, src_bf16);
    MXH_LAUNCH_CHECK("col_reduce");
}

// Folds [outer, chunks, S] f32 partials.  Many chunks go through a second round of partials (the other half of the
// scratch slot) so that the fold itself has enough threads.
template <class TOut, class R>
void fold_partials(const float* part, TOut* out, size_t outer, unsigned chunks, size_t S, float div, bool src_bf16) {
    size_t base_blocks = (outer * (S / 4 + 1) + RB - 1) / RB;
    if (chunks >= 64 && base_blocks < 64) {
        unsigned c2 = 8;
        size_t len2 = (chunks + c2 - 1) / c2;
        c2 = (unsigned)((chunks + len2 - 1) / len2);
        float* part2 = (float*)part + outer * (size_t)chunks * S + 64;
        col_stage<float, float, R>(part, part2, outer, chunks, S, c2, len2, 0.0f, src_bf16);
        col_stage<float, TOut, R>(part2, out, outer, c2, S, 1, c2, div, src_bf16);
        return;
    }
    col_stage<float, TOut, R>(part, out, outer, chunks, S, 1, chunks, div, src_bf16);
}

// The split kernel: 16 waves deep.  False when the shape does not fit it.
template <class TIn, class TOut, class R>
bool col_split_stage(const TIn* in, TOut* out, size_t outer, size_t L, size_t S, unsigned chunks, size_t chunk_len, float div,
                     bool src_bf16) {
    constexpr int VI = 16 / sizeof(TIn), VO = 16 / sizeof(TOut);
    constexpr int VEC = VI < VO ? VI : VO;
    constexpr int NW = 16;
    if (S % VEC != 0 || ((uintptr_t)in % (VEC * sizeof(TIn))) != 0 || ((uintptr_t)out % (VEC * sizeof(TOut))) != 0) return false;
    size_t sv = S / VEC, jblocks = cdiv(sv, (size_t)WAVE);
    size_t blocks = outer * chunks * jblocks;
    if (blocks >= (1ull << 31) || sv >= (1ull << 31)) return false;
    if (streams(outer * L * S * sizeof(TIn)))
        hipLaunchKernelGGL((col_reduce_split_kernel<TIn, TOut, R, VEC, NW, true>), dim3((unsigned)blocks), dim3(WAVE * NW), 0, stream(), in, out,
                           L, S, (uint32_t)sv, chunks, chunk_len, make_fastdiv((uint32_t)jblocks), make_fastdiv(chunks), div, src_bf16);
    else
        hipLaunchKernelGGL((col_reduce_split_kernel<TIn, TOut, R, VEC, NW>), dim3((unsigned)blocks), dim3(WAVE * NW), 0, stream(), in, out,
                           L, S, (uint32_t)sv, chunks, chunk_len, make_fastdiv((uint32_t)jblocks), make_fastdiv(chunks), div, src_bf16);
    MXH_LAUNCH_CHECK("col_reduce_split");
    return true;
}

// [outer, L, S] (contiguous) → out[outer, S]
template <class TIn, class TOut, class R>
void col_reduce(const TIn* in, TOut* out, size_t outer, size_t L, size_t S, float div, bool src_bf16) {
    // Narrow rows under a long axis (the gradient of a 5-element bias over 16 M rows): a thread per column would be five
    // threads.  G rows at a time are one wide row: [L, S] is read as [L / G, G * S], reduced to G * S partial columns by
    // the wide-row kernels below, and those G partial rows (plus one for the L % G rows left over, when there is one
    // slice) are folded by a second, small call.  [16777216, 5]: 2600 -> about 60 us.
    if (S < 64 && L >= 8192 && (t_fixed || !capture_open())) {
        size_t G = 256;
        if (outer > 1) while (G > 1 && L % G != 0) G /= 2;         // slices must stay whole
        const size_t L0 = L / G * G, rem = L - L0;
        if (G >= 8 && G * S >= 256) {
            float* P = regroup_rows(outer * (G + 1) * S * sizeof(float) + 256);
            if (!P) return;
            col_reduce<TIn, float, R>(in, P, outer, L0 / G, G * S, 0.0f, src_bf16);
            if (rem) col_reduce<TIn, float, R>(in + L0 * S, P + G * S, 1, rem, S, 0.0f, src_bf16);      // (outer == 1)
            col_reduce<float, TOut, R>(P, out, outer, G + (rem ? 1 : 0), S, div, src_bf16);
            return;
        }
    }
    {
        // wide rows and a long axis: blocks of 16 waves that split the axis among their waves
        constexpr int VI = 16 / sizeof(TIn), VO = 16 / sizeof(TOut);
        constexpr int VEC = VI < VO ? VI : VO;
        const size_t jblocks = cdiv(S / VEC, (size_t)WAVE);
        if (S % VEC == 0 && S / VEC >= WAVE && L >= 256) {
            size_t base = outer * jblocks;
            unsigned chunks = 1;
            if (base < COL_SPLIT_BLOCKS) chunks = (unsigned)std::min<size_t>(cdiv((size_t)COL_SPLIT_BLOCKS, base), L / 256);
            if (chunks < 1) chunks = 1;
            size_t chunk_len = cdiv(L, (size_t)chunks);
            chunks = (unsigned)cdiv(L, chunk_len);
            if (chunks == 1) {
                if (col_split_stage<TIn, TOut, R>(in, out, outer, L, S, 1, L, div, src_bf16)) return;
            } else {
                float* part = partials((outer * chunks * S + outer * 8 * S) * sizeof(float) + 1024);
                if (!part) return;
                if (col_split_stage<TIn, float, R>(in, part, outer, L, S, chunks, chunk_len, 0.0f, src_bf16)) {
                    fold_partials<TOut, R>(part, out, outer, chunks, S, div, src_bf16);
                    return;
                }
            }
        }
    }
    size_t base_blocks = (outer * (S / 4 + 1) + RB - 1) / RB;
    unsigned chunks = 1;
    size_t chunk_len = L;
    if (base_blocks < COL_TARGET_BLOCKS && L >= 2 * COL_MIN_ROWS) {
        size_t want = (COL_TARGET_BLOCKS + base_blocks - 1) / base_blocks;
        size_t max_chunks = L / COL_MIN_ROWS;   // at least this many rows per chunk
        chunks = (unsigned)(want < max_chunks ? want : max_chunks);
        if (chunks < 1) chunks = 1;
        chunk_len = (L + chunks - 1) / chunks;
        chunks = (unsigned)((L + chunk_len - 1) / chunk_len);
    }
    if (chunks == 1) { col_stage<TIn, TOut, R>(in, out, outer, L, S, 1, L, div, src_bf16); return; }
    float* part = partials((outer * chunks * S + outer * 8 * S) * sizeof(float) + 1024);
    if (!part) return;
    col_stage<TIn, float, R>(in, part, outer, L, S, chunks, chunk_len, 0.0f, src_bf16);
    fold_partials<TOut, R>(part, out, outer, chunks, S, div, src_bf16);
}

// [A, K, S] (contiguous) → out[K], both outer axes summed.  False when the shape does not fit the kernel.
template <class T>
bool plane_reduce(const T* in, T* out, size_t A, size_t K, size_t S) {
    constexpr int VEC = 16 / sizeof(T);
    if (S % VEC != 0 || !aligned16(in) || A * (S / VEC) >= (1ull << 31) || K >= (1ull << 24) || A >= (1ull << 31) || S >= (1ull << 31)) return false;
    if (A * (S / VEC) < 2 * PLB) return false;         // too little per block to be worth it
    // one block per kept index when there are enough of them, else cut the rows into chunks
    uint32_t chunks = 1;
    if (K < 256) chunks = (uint32_t)std::min<size_t>(A, cdiv((size_t)512, K));
    uint32_t a_chunk = (uint32_t)cdiv(A, (size_t)chunks);
    chunks = (uint32_t)cdiv(A, (size_t)a_chunk);
    if (K * chunks >= (1ull << 31)) return false;
    FastDiv dsv = make_fastdiv((uint32_t)(S / VEC));
    const bool bf = IO<T>::is_bf16;
    if (chunks == 1) {
        hipLaunchKernelGGL((plane_reduce_kernel<T, T, RSum, VEC, true>), dim3((unsigned)K), dim3(PLB), 0, stream(), in, out, (uint32_t)A,
                           (uint32_t)K, (uint32_t)S, a_chunk, dsv, bf);
        MXH_LAUNCH_CHECK("plane_reduce");
        return true;
    }
    float* part = partials(((size_t)chunks * K + 8 * K) * sizeof(float) + 1024);
    if (!part) return true;      // status is set
    hipLaunchKernelGGL((plane_reduce_kernel<T, float, RSum, VEC, true>), dim3((unsigned)(K * chunks)), dim3(PLB), 0, stream(), in, part,
                       (uint32_t)A, (uint32_t)K, (uint32_t)S, a_chunk, dsv, bf);
    MXH_LAUNCH_CHECK("plane_reduce");
    fold_partials<T, RSum>(part, out, 1, chunks, K, 0.0f, bf);
    return true;
}

// sum/mean/max/min metadata: dims[n] | strides[n] | red_len[r] | red_stride[r] | offset
template <class T, class R>
void reduce_axis(size_t num_els, size_t num_dims, size_t nred, const size_t* md, const T* in, T* out, bool mean) {
    if (!md || !in || !out) { set_status(ERR_INVALID, "reduce: null argument"); return; }
    if (nred != 1) { set_status(ERR_UNSUPPORTED, "reduce: exactly one reduced dim is supported"); return; }
    if (num_els == 0) return;
    const size_t* dims = md;
    const size_t* strides = md + num_dims;
    size_t L = md[2 * num_dims], s = md[2 * num_dims + 1], offset = md[2 * num_dims + 2];
    if (L == 0) { set_status(ERR_INVALID, "reduce: zero-length axis"); return; }
    float div = mean ? (float)L : 0.0f;
    const T* src = in + offset;
    size_t out_size = num_els / L;
    if (out_size == 0) return;
    if (ref_is_contiguous(num_dims, dims, strides) && s != 0 && num_els % (L * s) == 0) {
        size_t outer = num_els / (L * s);
        if (s == 1) row_reduce<T, T, R>(src, out, outer, L, div, IO<T>::is_bf16);
        else col_reduce<T, T, R>(src, out, outer, L, s, div, IO<T>::is_bf16);
        return;
    }
    if (num_els >= (1ull << 31)) { set_status(ERR_TOO_LARGE, "reduce: strided input with 2^31 or more elements"); return; }
    // A large strided input whose logical index space divides into whole slices: the reference reduces the logical
    // layout [outer, L, s] with every element fetched through get_strided_index (reduction.rs:728-729 hands over the
    // memory stride of the reduced dim as s, and that is what is reproduced).  Copied into logical order first - the
    // elementwise identity walks the view by exactly that index rule, and has a tiled kernel for transposed views -
    // it is the contiguous reduction of the copy: [8192,8192] viewed transposed 3900 -> about 160 us.  (Not while a
    // capture is open, where the scratch block cannot grow; small inputs keep the one-thread-per-output kernel.)
    {
        const size_t se = s != 0 ? s : 1;          // s = 0: logical index d * L + l, the layout [out_size, L]
        if (num_els >= (1u << 18) && num_dims <= 64 && num_els % (L * se) == 0 && !capture_open() && !t_fixed) {
            T* tmp = (T*)scratch(num_els * sizeof(T), 1);
            if (!tmp) return;                      // status is set
            size_t cs[64];
            contiguous_strides(num_dims, dims, cs);
            const size_t* ins[1] = {strides};
            const void* inp[1] = {src};
            ew_launch<OpIdentity<T>>(num_els, num_dims, dims, cs, ins, tmp, inp, OpIdentity<T>{});
            const size_t outer = num_els / (L * se);
            if (se == 1) row_reduce<T, T, R>(tmp, out, outer, L, div, IO<T>::is_bf16);
            else col_reduce<T, T, R>(tmp, out, outer, L, se, div, IO<T>::is_bf16);
            return;
        }
    }
    NdSpace<1> sp;
    // not collapsed on purpose: the walk must visit dims exactly as get_strided_index does
    if (num_dims > (size_t)MAXD) { set_status(ERR_UNSUPPORTED, "reduce: strided input of rank above 8"); return; }
    sp.ndims = (int)(num_dims ? num_dims : 1);
    for (int d = 0; d < MAXD; ++d) {
        sp.dims[d] = d < (int)num_dims ? (uint32_t)dims[d] : 1;
        sp.div[d] = make_fastdiv(sp.dims[d]);
        sp.strides[0][d] = d < (int)num_dims ? (int64_t)strides[d] : 0;
    }
    hipLaunchKernelGGL((reduce_generic_kernel<T, R>), dim3(cdiv(out_size, RB)), dim3(RB), 0, stream(), sp, src, out, num_els,
                       out_size, L, s, div);
    MXH_LAUNCH_CHECK("reduce_generic");
}

// ---- sum_to_shape -----------------------------------------------------------------------------------

// Non-contiguous input: gather into a contiguous copy with the reference's index rule
// (reduction.rs:162-167): element (Σ coords·strides + offset) mod num_els of the already-offset slice.
template <class T>
__global__ __launch_bounds__(RB) void sts_gather_kernel(NdSpace<1> sp, const T* __restrict__ in, T* __restrict__ out,
                                                        size_t num_els, size_t offset) {
    size_t i = (size_t)blockIdx.x * RB + threadIdx.x;
    if (i >= num_els) return;
    uint32_t r = (uint32_t)i;
    uint64_t off = 0;
    for (int k = sp.ndims - 1; k > 0; --k) {
        uint32_t q, c;
        fd_divmod(r, sp.div[k], q, c);
        off += (uint64_t)c * (uint64_t)sp.strides[0][k];
        r = q;
    }
    off += (uint64_t)r * (uint64_t)sp.strides[0][0];
    out[i] = in[(off + offset) % num_els];
}

// sum_to_shape metadata: in_dims[n] | in_strides[n] | out_dims[n] | offset
template <class T>
void sum_to_shape(size_t num_els, size_t num_dims, const size_t* md, const T* in, T* out) {
    if (!md || !in || !out) { set_status(ERR_INVALID, "sum_to_shape: null argument"); return; }
    if (num_els == 0) return;
    if (num_dims > 64) { set_status(ERR_INVALID, "sum_to_shape: rank above 64"); return; }
    const size_t* in_dims = md;
    const size_t* in_strides = md + num_dims;
    const size_t* out_dims = md + 2 * num_dims;
    size_t offset = md[3 * num_dims];
    const T* src = in + offset;

    // groups of kept (factor 1) and reduced (factor = whole dim) dims; size-1 dims vanish
    size_t g_len[64];
    bool g_red[64];
    int ng = 0;
    for (size_t d = 0; d < num_dims; ++d) {
        if (out_dims[d] == 0 || in_dims[d] % out_dims[d] != 0 || (out_dims[d] != 1 && out_dims[d] != in_dims[d])) {
            set_status(ERR_UNSUPPORTED, "sum_to_shape: output dim must be 1 or the input dim");
            return;
        }
        if (in_dims[d] == 1) continue;
        bool red = out_dims[d] == 1;
        if (ng > 0 && g_red[ng - 1] == red) g_len[ng - 1] *= in_dims[d];
        else { g_len[ng] = in_dims[d]; g_red[ng] = red; ++ng; }
    }

    bool cont = ref_is_contiguous(num_dims, in_dims, in_strides);
    bool any_red = false;
    int nred_groups = 0;
    for (int g = 0; g < ng; ++g) { any_red |= g_red[g]; nred_groups += g_red[g]; }
    if (!cont && !any_red) {
        // identity on a strided view (a broadcast gradient being accumulated for the first time): when no source index
        // reaches num_els the reference's wrap-around (see sts_gather_kernel) never applies, and out = 0 + view is one
        // elementwise pass over the view's own strides instead of a gathered copy followed by that pass
        size_t last = offset;
        for (size_t d = 0; d < num_dims; ++d) last += (in_dims[d] - 1) * in_strides[d];
        if (last < num_els) {
            size_t cs[64];
            contiguous_strides(num_dims, in_dims, cs);
            const size_t* ins[1] = {in_strides};
            const void* inp[1] = {src + offset};
            ew_launch<OpZeroPlus<T>>(num_els, num_dims, in_dims, cs, ins, out, inp, OpZeroPlus<T>{});
            return;
        }
    }
    // Temporaries (slot 1 of the library scratch; the stage drivers' partials use slot 0):
    // [gathered contiguous copy | ping | pong]
    T* gathered = nullptr;
    float *ping = nullptr, *pong = nullptr;
    size_t gathered_bytes = cont ? 0 : (num_els * sizeof(T) + 255) / 256 * 256;
    size_t stage_bytes = 0;
    if (nred_groups > 1) {
        size_t smallest = (size_t)-1;
        for (int g = 0; g < ng; ++g) if (g_red[g] && g_len[g] < smallest) smallest = g_len[g];
        stage_bytes = ((num_els / smallest) * sizeof(float) + 255) / 256 * 256;
    }
    if (gathered_bytes + 2 * stage_bytes) {
        char* p = (char*)scratch(gathered_bytes + 2 * stage_bytes, 1);
        if (!p) return;
        if (!cont) { gathered = (T*)p; p += gathered_bytes; }
        if (stage_bytes) { ping = (float*)p; pong = (float*)(p + stage_bytes); }
    }
    if (!cont) {
        if (num_els >= (1ull << 31) || num_dims > (size_t)MAXD) {
            set_status(ERR_UNSUPPORTED, "sum_to_shape: strided input too large or rank above 8");
            return;
        }
        size_t last = offset;
        for (size_t d = 0; d < num_dims; ++d) last += (in_dims[d] - 1) * in_strides[d];
        if (last < num_els) {
            // no source index reaches num_els, so the wrap-around of the reference's rule never applies: the copy is the
            // elementwise identity over the view (tiled for transposed views; a [8192,8192] one: 320 -> 110 us)
            size_t cs[64];
            contiguous_strides(num_dims, in_dims, cs);
            const size_t* ins[1] = {in_strides};
            const void* inp[1] = {src + offset};
            ew_launch<OpIdentity<T>>(num_els, num_dims, in_dims, cs, ins, gathered, inp, OpIdentity<T>{});
        } else {
            NdSpace<1> sp;
            sp.ndims = (int)(num_dims ? num_dims : 1);
            for (int d = 0; d < MAXD; ++d) {
                sp.dims[d] = d < (int)num_dims ? (uint32_t)in_dims[d] : 1;
                sp.div[d] = make_fastdiv(sp.dims[d]);
                sp.strides[0][d] = d < (int)num_dims ? (int64_t)in_strides[d] : 0;
            }
            hipLaunchKernelGGL((sts_gather_kernel<T>), dim3(cdiv(num_els, RB)), dim3(RB), 0, stream(), sp, src, gathered, num_els,
                               offset);
            MXH_LAUNCH_CHECK("sts_gather");
        }
        src = gathered;
    }

    if (!any_red) {   // identity: out = 0 + in
        size_t dims1 = num_els, st1 = 1;
        const size_t* ins[1] = {&st1};
        const void* inp[1] = {src};
        ew_launch<OpZeroPlus<T>>(num_els, 1, &dims1, &st1, ins, out, inp, OpZeroPlus<T>{});
    } else if (ng == 3 && g_red[0] && !g_red[1] && g_red[2] && plane_reduce<T>(src, out, g_len[0], g_len[1], g_len[2])) {
        // [reduced, kept, reduced] in one pass
    } else {
        // fold reduced groups one at a time, innermost first
        const void* cur = src;
        bool cur_is_T = true;
        while (true) {
            int g = ng - 1;
            while (!g_red[g]) --g;
            size_t outer = 1, inner = 1;
            for (int k = 0; k < g; ++k) outer *= g_len[k];
            for (int k = g + 1; k < ng; ++k) inner *= g_len[k];
            size_t L = g_len[g];
            int remaining = 0;
            for (int k = 0; k < ng; ++k) remaining += (k != g && g_red[k]);
            bool last = remaining == 0;
            float* tmp = (cur == (const void*)ping) ? pong : ping;
            bool bf = IO<T>::is_bf16;
            if (inner == 1) {
                if (cur_is_T) { if (last) row_reduce<T, T, RSum>((const T*)cur, out, outer, L, 0.0f, bf); else row_reduce<T, float, RSum>((const T*)cur, tmp, outer, L, 0.0f, bf); }
                else { if (last) row_reduce<float, T, RSum>((const float*)cur, out, outer, L, 0.0f, bf); else row_reduce<float, float, RSum>((const float*)cur, tmp, outer, L, 0.0f, bf); }
            } else {
                if (cur_is_T) { if (last) col_reduce<T, T, RSum>((const T*)cur, out, outer, L, inner, 0.0f, bf); else col_reduce<T, float, RSum>((const T*)cur, tmp, outer, L, inner, 0.0f, bf); }
                else { if (last) col_reduce<float, T, RSum>((const float*)cur, out, outer, L, inner, 0.0f, bf); else col_reduce<float, float, RSum>((const float*)cur, tmp, outer, L, inner, 0.0f, bf); }
            }
            if (last) break;
            cur = tmp;
            cur_is_T = false;
            // drop group g and merge its neighbours (both kept) if both exist
            for (int k = g; k + 1 < ng; ++k) { g_len[k] = g_len[k + 1]; g_red[k] = g_red[k + 1]; }
            --ng;
            if (g > 0 && g < ng && g_red[g - 1] == g_red[g]) {
                g_len[g - 1] *= g_len[g];
                for (int k = g; k + 1 < ng; ++k) { g_len[k] = g_len[k + 1]; g_red[k] = g_red[k + 1]; }
                --ng;
            }
        }
    }
}

// ---- fold ---------------------------------------------------------------------------------------------
// The adjoint of unfold (crates/maidenx_cpu/src/ops/reduction.rs:274-380): input element c adds to the
// output at c without the window dim and with the fold dim set to c[fold]*step + c[window].  Gather
// form: one thread per output element sums its windows in ascending order in f32 (the reference adds
// in scheduling order in the storage dtype).  The source index is (sum c*stride) % num_els (:336-340).
// metadata: dims[n] | strides[n] | fold_dim, window_dim, fold_size, step, window_size, offset
struct FoldSpace {
    int nd_out;                      // output rank (input rank - 1)
    int fold_slot;                   // position of the folded dim among the output dims
    uint32_t out_dims[MAXD];
    FastDiv div[MAXD];
    int64_t strides[MAXD];           // input stride of each output dim (the fold slot: unused)
    int64_t fold_stride, window_stride;
    uint32_t n_windows, window, step;
};

// The type a fold's sums are formed in: f32 for the 32- and 16-bit floats (one rounding at the end), f64 for f64, the
// unsigned counterpart for the integers (wrapping, as the reference's release build; its debug build panics).
template <class T, class = void> struct FoldAcc {
    using A = float;
    static __device__ A ld(T v) { return IO<T>::ld(v); }
    static __device__ T st(A a) { return IO<T>::fin(a, 0.0f); }
};
template <> struct FoldAcc<double, void> {
    using A = double;
    static __device__ A ld(double v) { return v; }
    static __device__ double st(A a) { return a; }
};
template <class T> struct FoldAcc<T, typename std::enable_if<std::is_integral<T>::value>::type> {
    using A = typename std::make_unsigned<T>::type;
    static __device__ A ld(T v) { return (A)v; }
    static __device__ T st(A a) { return (T)a; }
};

template <class T>
__global__ __launch_bounds__(RB) void fold_kernel(FoldSpace sp, const T* __restrict__ in, T* __restrict__ out, size_t out_size,
                                                  size_t num_els) {
    size_t o = (size_t)blockIdx.x * RB + threadIdx.x;
    if (o >= out_size) return;
    uint32_t r = (uint32_t)o, p = 0;
    int64_t base = 0;
#pragma unroll
    for (int d = MAXD - 1; d >= 0; --d) {
        if (d >= sp.nd_out) continue;
        uint32_t q, c;
        if (d > 0) fd_divmod(r, sp.div[d], q, c);
        else { q = 0; c = r; }
        if (d == sp.fold_slot) p = c;
        else base += (int64_t)c * sp.strides[d];
        r = q;
    }
    using FA = FoldAcc<T>;
    typename FA::A acc = 0;
    if (sp.step == 0) {
        if (p < sp.window)
            for (uint32_t w = 0; w < sp.n_windows; ++w)
                acc = acc + FA::ld(in[(uint64_t)(base + (int64_t)w * sp.fold_stride + (int64_t)p * sp.window_stride) % num_els]);
    } else {
        uint32_t w0 = p >= sp.window ? (p - sp.window) / sp.step + 1 : 0;
        uint32_t w1 = p / sp.step;
        if (w1 >= sp.n_windows) w1 = sp.n_windows - 1;
        for (uint32_t w = w0; w <= w1 && sp.n_windows > 0; ++w) {
            uint32_t pos = p - w * sp.step;
            acc = acc + FA::ld(in[(uint64_t)(base + (int64_t)w * sp.fold_stride + (int64_t)pos * sp.window_stride) % num_els]);
        }
    }
    out[o] = FA::st(acc);
}

template <class T>
void fold(size_t num_els, size_t nd, const size_t* md, const T* in, T* out) {
    if (!md || !in || !out) { set_status(ERR_INVALID, "fold: null argument"); return; }
    if (nd < 2 || nd > (size_t)MAXD + 1) { set_status(ERR_UNSUPPORTED, "fold: rank must be 2..9"); return; }
    const size_t* dims = md;
    const size_t* strides = md + nd;
    const size_t fold_dim = md[2 * nd], window_dim = md[2 * nd + 1], fold_size = md[2 * nd + 2], step = md[2 * nd + 3];
    const size_t offset = md[2 * nd + 5];
    if (fold_dim >= nd || window_dim >= nd || fold_dim == window_dim) { set_status(ERR_INVALID, "fold: bad dims"); return; }
    FoldSpace sp;
    size_t out_size = 1;
    int k = 0;
    sp.fold_slot = 0;
    for (size_t d = 0; d < nd; ++d) {
        if (d == window_dim) continue;
        size_t len = d == fold_dim ? fold_size : dims[d];
        if (d == fold_dim) sp.fold_slot = k;
        sp.out_dims[k] = (uint32_t)len;
        sp.div[k] = make_fastdiv((uint32_t)len);
        sp.strides[k] = (int64_t)strides[d];
        out_size *= len;
        ++k;
    }
    sp.nd_out = k;
    for (; k < MAXD; ++k) { sp.out_dims[k] = 1; sp.div[k] = make_fastdiv(1); sp.strides[k] = 0; }
    if (out_size == 0) return;
    if (out_size >= (1ull << 31) || num_els >= (1ull << 31) || step >= (1ull << 31)) { set_status(ERR_TOO_LARGE, "fold: 2^31 or more elements"); return; }
    if (num_els == 0) { set_status(ERR_INVALID, "fold: empty input"); return; }
    sp.fold_stride = (int64_t)strides[fold_dim];
    sp.window_stride = (int64_t)strides[window_dim];
    sp.n_windows = (uint32_t)dims[fold_dim];
    sp.window = (uint32_t)dims[window_dim];
    sp.step = (uint32_t)step;
    hipLaunchKernelGGL(fold_kernel<T>, dim3(cdiv(out_size, RB)), dim3(RB), 0, stream(), sp, in + offset, out, out_size, num_els);
    MXH_LAUNCH_CHECK("fold");
}

}  // namespace mxh

using namespace mxh;

#define MXH_REDUCE_FOR(T, SUF)                                                                                  \
    extern "C" void hip_sum_##SUF(size_t n, size_t nd, size_t nr, const size_t* md, const T* in, T* out) { MXH_API; \
        reduce_axis<T, RSum>(n, nd, nr, md, in, out, false);                                                    \
    }                                                                                                           \
    extern "C" void hip_mean_##SUF(size_t n, size_t nd, size_t nr, const size_t* md, const T* in, T* out) { MXH_API; \
        reduce_axis<T, RSum>(n, nd, nr, md, in, out, true);                                                     \
    }                                                                                                           \
    extern "C" void hip_max_##SUF(size_t n, size_t nd, size_t nr, const size_t* md, const T* in, T* out) { MXH_API; \
        reduce_axis<T, RMax>(n, nd, nr, md, in, out, false);                                                    \
    }                                                                                                           \
    extern "C" void hip_min_##SUF(size_t n, size_t nd, size_t nr, const size_t* md, const T* in, T* out) { MXH_API; \
        reduce_axis<T, RMin>(n, nd, nr, md, in, out, false);                                                    \
    }                                                                                                           \
    extern "C" void hip_sum_to_shape_##SUF(size_t n, size_t nd, const size_t* md, const T* in, T* out) { MXH_API; \
        sum_to_shape<T>(n, nd, md, in, out);                                                                    \
    }                                                                                                           \
    extern "C" void hip_fold_##SUF(size_t n, size_t nd, const size_t* md, const T* in, T* out) { MXH_API;       \
        fold<T>(n, nd, md, in, out);                                                                            \
    }

MXH_REDUCE_FOR(float, f32)
MXH_REDUCE_FOR(bf16_t, bf16)
MXH_REDUCE_FOR(f16_t, f16)

// fold for f64 and the integers (crates/maidenx_cuda/src/ops/reduction.rs:44-93 lists `fold` for every dtype; CPU
// instantiations at crates/maidenx_cpu/src/ops/reduction.rs:632-643).  Their other reductions are in reduce_wide.hip.
#define MXH_FOLD_FOR(T, SUF)                                                                                    \
    extern "C" void hip_fold_##SUF(size_t n, size_t nd, const size_t* md, const T* in, T* out) { MXH_API;       \
        fold<T>(n, nd, md, in, out);                                                                            \
    }
MXH_FOLD_FOR(double, f64)
MXH_FOLD_FOR(uint8_t, u8)
MXH_FOLD_FOR(uint16_t, u16)
MXH_FOLD_FOR(uint32_t, u32)
MXH_FOLD_FOR(uint64_t, u64)
MXH_FOLD_FOR(int8_t, i8)
MXH_FOLD_FOR(int16_t, i16)
MXH_FOLD_FOR(int32_t, i32)
MXH_FOLD_FOR(int64_t, i64)

// hip_sum_f32 for callers that cannot allocate (under graph capture, in a serving loop, in a harness that forbids it):
// same arguments and kernels, but chunk partials and regrouped partial rows go to the fixed array above instead of the
// library's grown-on-demand scratch, so the call performs no hipMalloc / hipFree / stream synchronisation whatever ran
// before it.  For a contiguous input the result has the bits of hip_sum_f32 (outside a capture).  A strided input is
// never copied into logical order here (that copy lives in grown scratch): it is summed one thread per output in
// ascending order, the reference's sequential order, which agrees with hip_sum_f32's tree to rounding only.  A shape
// whose partials exceed their part of the array is refused (status ERR_TOO_LARGE) and nothing is queued.  Every partial a launch reads was written
// by the launch before it, so nothing needs clearing between calls; all calls on a device share that device's array,
// so calls that overlap on one device (two streams, two threads that switch streams) race.
extern "C" void hip_sum_f32_noalloc(size_t n, size_t nd, size_t nr, const size_t* md, const float* in, float* out) { MXH_API;
    void* p = fixed_partials();
    if (!p) return;
    t_fixed = p;
    reduce_axis<float, RSum>(n, nd, nr, md, in, out, false);
    t_fixed = nullptr;
}
// Resolves the array's address on the current device ahead of time (optional: the first hip_sum_f32_noalloc does it too).
extern "C" int hip_noalloc_prepare(void) { MXH_API_INT; return fixed_partials() ? 0 : (int)hipErrorInvalidSymbol; }
