// sum / max / min (f64 also mean) along one axis and sum_to_shape for f64 and the integer dtypes
// (crates/maidenx_cuda/src/ops/reduction.rs:59-113 of the reference's declarations; semantics
// crates/maidenx_cpu/src/ops/reduction.rs:6-89 sum, :185-272 mean, :383-553 max / min, :91-183 sum_to_shape).
// For these dtypes the accumulator is the storage type itself, so partial results are plain T: integer sums wrap (the
// reference's release build; its debug build panics on overflow), which makes them independent of the order of
// addition - any tree gives the reference's bits; max / min are order-independent; f64 sums differ from the reference's
// sequential order by rounding only.
#include <cfloat>

#include "elementwise.hpp"
#include "ops.hpp"
#include "mxh.hpp"

namespace mxh {

bool capture_open();      // runtime.hip: a graph capture is being recorded


constexpr int WB = 256;

struct WSum {
    template <class T> static __device__ T init() { return (T)0; }
    template <class T> static __device__ T op(T a, T b) {
        if constexpr (std::is_integral<T>::value) {
            using U = typename std::make_unsigned<T>::type;
            return (T)(U)((U)a + (U)b);
        } else return a + b;
    }
};
// `if val > out { val } else { out }` from the type's MIN (f64::MIN = -DBL_MAX): a NaN never wins
struct WMax {
    template <class T> static __device__ T init() { return std::numeric_limits<T>::lowest(); }
    template <class T> static __device__ T op(T a, T b) { return b > a ? b : a; }
};
struct WMin {
    template <class T> static __device__ T init() { return std::numeric_limits<T>::max(); }
    template <class T> static __device__ T op(T a, T b) { return b < a ? b : a; }
};
// the mean's single division at the end (reduction.rs:264-268); div == 0: none
template <class T> __device__ inline T wfin(T acc, double div) {
    if constexpr (std::is_same<T, double>::value) return div != 0.0 ? acc / div : acc;
    else return acc;
}

// ---- [rows, L] -> [rows, chunks]: one block per (row, chunk) ---------------------------------------------------------
// VEC > 1 needs L % VEC == 0, chunk_len % VEC == 0 and a 16-byte aligned base.  Four loads in flight per thread.
template <class T, class R, int VEC>
__global__ __launch_bounds__(WB) void wrow_kernel(const T* __restrict__ in, T* __restrict__ out, size_t L, unsigned chunks, size_t chunk_len,
                                                  double div) {
    const size_t row = blockIdx.x / chunks, chunk = blockIdx.x % chunks;
    const size_t beg = chunk * chunk_len, end = beg + chunk_len < L ? beg + chunk_len : L;
    const T* src = in + row * L;
    T a[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) a[e] = R::template init<T>();
    constexpr size_t STEP = (size_t)WB * VEC;
    size_t i = beg + (size_t)threadIdx.x * VEC;
    for (; i + 3 * STEP < end; i += 4 * STEP) {
        AVec<T, VEC> v[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) v[k] = *(const AVec<T, VEC>*)(src + i + k * STEP);
#pragma unroll
        for (int k = 0; k < 4; ++k)
#pragma unroll
            for (int e = 0; e < VEC; ++e) a[e] = R::op(a[e], v[k].v[e]);
    }
    for (; i < end; i += STEP) {
        AVec<T, VEC> v = *(const AVec<T, VEC>*)(src + i);
#pragma unroll
        for (int e = 0; e < VEC; ++e) a[e] = R::op(a[e], v.v[e]);
    }
    T acc = a[0];
#pragma unroll
    for (int e = 1; e < VEC; ++e) acc = R::op(acc, a[e]);
    __shared__ T part[WB];
    part[threadIdx.x] = acc;
    __syncthreads();
#pragma unroll
    for (int s = WB / 2; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) part[threadIdx.x] = R::op(part[threadIdx.x], part[threadIdx.x + s]);
        __syncthreads();
    }
    if (threadIdx.x == 0) out[blockIdx.x] = wfin(part[0], div);
}

// ---- [outer, L, S] -> [outer, chunks, S]: one thread per (o, chunk, column vector), coalesced across the columns ------
template <class T, class R, int VEC>
__global__ __launch_bounds__(WB) void wcol_kernel(const T* __restrict__ in, T* __restrict__ out, size_t L, size_t S, unsigned chunks,
                                                  size_t chunk_len, FastDiv div_sv, FastDiv div_chunks, size_t total, double div) {
    const size_t tid = (size_t)blockIdx.x * WB + threadIdx.x;
    if (tid >= total) return;
    uint32_t rest, jv, o, chunk;
    fd_divmod((uint32_t)tid, div_sv, rest, jv);
    fd_divmod(rest, div_chunks, o, chunk);
    const size_t beg = (size_t)chunk * chunk_len, end = beg + chunk_len < L ? beg + chunk_len : L;
    const T* src = in + ((size_t)o * L + beg) * S + (size_t)jv * VEC;
    T a[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) a[e] = R::template init<T>();
    size_t l = beg;
    for (; l + 8 <= end; l += 8, src += 8 * S) {
        AVec<T, VEC> v[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) v[k] = *(const AVec<T, VEC>*)(src + k * S);
#pragma unroll
        for (int k = 0; k < 8; ++k)
#pragma unroll
            for (int e = 0; e < VEC; ++e) a[e] = R::op(a[e], v[k].v[e]);
    }
    for (; l < end; ++l, src += S) {
        AVec<T, VEC> v = *(const AVec<T, VEC>*)src;
#pragma unroll
        for (int e = 0; e < VEC; ++e) a[e] = R::op(a[e], v.v[e]);
    }
    AVec<T, VEC> r;
#pragma unroll
    for (int e = 0; e < VEC; ++e) r.v[e] = wfin(a[e], div);
    *(AVec<T, VEC>*)(out + ((size_t)o * chunks + chunk) * S + (size_t)jv * VEC) = r;
}

// ---- [outer, L, S] -> [outer, chunks, S] with the axis split inside the block -------------------------------------------
// A block is NW waves deep: wave w walks slice w of the chunk's rows for the same 64 column vectors with eight loads in
// flight per lane, and the NW partial rows meet in LDS in wave order: the loads in flight of NW threads per column
// without NW times the partials.  Needs S % VEC == 0 and aligned bases.
template <class T, class R, int VEC, int NW>
__global__ __launch_bounds__(WAVE * NW) void wcol_split_kernel(const T* __restrict__ in, T* __restrict__ out, size_t L, size_t S, uint32_t sv,
                                                                unsigned chunks, size_t chunk_len, FastDiv div_jb, FastDiv div_chunks, double div) {
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
    T a[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) a[e] = R::template init<T>();
    if (live) {
        const T* src = in + ((size_t)o * L + l0) * S + (size_t)jv * VEC;
        size_t l = l0;
        for (; l + U <= l1; l += U, src += U * S) {
            AVec<T, VEC> v[U];
#pragma unroll
            for (int k = 0; k < U; ++k) v[k] = *(const AVec<T, VEC>*)(src + k * S);
#pragma unroll
            for (int k = 0; k < U; ++k)
#pragma unroll
                for (int e = 0; e < VEC; ++e) a[e] = R::op(a[e], v[k].v[e]);
        }
        for (; l < l1; ++l, src += S) {
            AVec<T, VEC> v = *(const AVec<T, VEC>*)src;
#pragma unroll
            for (int e = 0; e < VEC; ++e) a[e] = R::op(a[e], v.v[e]);
        }
    }
    __shared__ T part[NW][VEC][WAVE];
#pragma unroll
    for (int e = 0; e < VEC; ++e) part[w][e][lane] = a[e];
    __syncthreads();
    if (w == 0 && live) {
        AVec<T, VEC> r;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            T t = part[0][e][lane];
#pragma unroll
            for (int k = 1; k < NW; ++k) t = R::op(t, part[k][e][lane]);
            r.v[e] = wfin(t, div);
        }
        *(AVec<T, VEC>*)(out + ((size_t)o * chunks + chunk) * S + (size_t)jv * VEC) = r;
    }
}

// ---- strided input: one thread per output element, indices as the reference's non-contiguous branch forms them -------
template <class T, class R>
__global__ __launch_bounds__(WB) void wgeneric_kernel(NdSpace<1> sp, const T* __restrict__ in, T* __restrict__ out, size_t num_els,
                                                      size_t out_size, size_t L, size_t s, double div) {
    const size_t d = (size_t)blockIdx.x * WB + threadIdx.x;
    if (d >= out_size) return;
    T acc = R::template init<T>();
    for (size_t l = 0; l < L; ++l) {
        const size_t i = s != 0 ? ((d / s) * L + l) * s + d % s : d * L + l;
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
        acc = R::op(acc, in[off]);
    }
    out[d] = wfin(acc, div);
}

template <class T, class R, int VEC>
static void wrow_launch(const T* in, T* out, size_t rows, size_t L, unsigned chunks, size_t chunk_len, double div) {
    hipLaunchKernelGGL((wrow_kernel<T, R, VEC>), dim3((unsigned)(rows * chunks)), dim3(WB), 0, stream(), in, out, L, chunks, chunk_len, div);
    MXH_LAUNCH_CHECK("reduce_wide_row");
}
template <class T, class R>
static void wrow_stage(const T* in, T* out, size_t rows, size_t L, unsigned chunks, size_t chunk_len, double div) {
    constexpr int V = 16 / sizeof(T);
    if (V > 1 && L % V == 0 && chunk_len % V == 0 && (uintptr_t)in % 16 == 0) wrow_launch<T, R, V>(in, out, rows, L, chunks, chunk_len, div);
    else wrow_launch<T, R, 1>(in, out, rows, L, chunks, chunk_len, div);
}
template <class T, class R>
static bool wcol_stage(const T* in, T* out, size_t outer, size_t L, size_t S, unsigned chunks, size_t chunk_len, double div) {
    constexpr int V = 16 / sizeof(T);
    const bool vec = V > 1 && S % V == 0 && (uintptr_t)in % 16 == 0 && (uintptr_t)out % 16 == 0;
    const size_t sv = vec ? S / V : S, total = outer * chunks * sv;
    if (total >= (1ull << 32) || sv >= (1ull << 32)) { set_status(ERR_TOO_LARGE, "reduce: 2^32 or more output columns"); return false; }
    const FastDiv dsv = make_fastdiv((uint32_t)sv), dch = make_fastdiv(chunks);
    if (vec) hipLaunchKernelGGL((wcol_kernel<T, R, V>), dim3((unsigned)cdiv(total, (size_t)WB)), dim3(WB), 0, stream(), in, out, L, S, chunks, chunk_len, dsv, dch, total, div);
    else hipLaunchKernelGGL((wcol_kernel<T, R, 1>), dim3((unsigned)cdiv(total, (size_t)WB)), dim3(WB), 0, stream(), in, out, L, S, chunks, chunk_len, dsv, dch, total, div);
    MXH_LAUNCH_CHECK("reduce_wide_col");
    return true;
}

// The split kernel, 16 waves deep.  False when the shape does not fit it (nothing launched then).
template <class T, class R>
static bool wcol_split_stage(const T* in, T* out, size_t outer, size_t L, size_t S, unsigned chunks, size_t chunk_len, double div) {
    constexpr int V = 16 / sizeof(T), NW = 16;
    if (S % V != 0 || (uintptr_t)in % 16 != 0 || (uintptr_t)out % 16 != 0) return false;
    const size_t sv = S / V, jblocks = cdiv(sv, (size_t)WAVE), blocks = outer * chunks * jblocks;
    if (blocks >= (1ull << 31) || sv >= (1ull << 31)) return false;
    hipLaunchKernelGGL((wcol_split_kernel<T, R, V, NW>), dim3((unsigned)blocks), dim3(WAVE * NW), 0, stream(), in, out, L, S, (uint32_t)sv, chunks,
                       chunk_len, make_fastdiv((uint32_t)jblocks), make_fastdiv(chunks), div);
    MXH_LAUNCH_CHECK("reduce_wide_col_split");
    return true;
}

// [outer, L, S] (contiguous) -> [outer, S].  Few outputs: the axis is cut into chunks whose partial results (plain T,
// in the library's scratch block) a second launch of the same kernels combines in chunk order.
template <class T, class R>
static void wreduce(const T* in, T* out, size_t outer, size_t L, size_t S, double div) {
    if (outer * S >= (1ull << 31)) { set_status(ERR_TOO_LARGE, "reduce: 2^31 or more outputs"); return; }
    if (S == 1) {
        const size_t per_block = (size_t)WB * (16 / sizeof(T)) * 8;          // what a block covers in two rounds of four loads
        size_t chunks = 1;
        if (outer < 1024 && L > per_block) {
            chunks = std::min<size_t>(cdiv((size_t)2048, outer), L / per_block);
            if (chunks < 1) chunks = 1;
        }
        size_t chunk_len = cdiv(L, chunks);
        chunk_len = cdiv(chunk_len, (size_t)64) * 64;                        // whole vectors
        chunks = cdiv(L, chunk_len);
        if (chunks == 1) { wrow_stage<T, R>(in, out, outer, L, 1, L, div); return; }
        T* part = (T*)scratch(outer * chunks * sizeof(T) + 256);
        if (!part) return;
        wrow_stage<T, R>(in, part, outer, L, (unsigned)chunks, chunk_len, 0.0);
        wrow_stage<T, R>(part, out, outer, chunks, 1, chunks, div);
        return;
    }
    // narrow rows under a long axis: G rows at a time as one wide row, the G partial rows (and the one of the left-over
    // rows, when there is one slice) folded by a second call - see col_reduce in reduce.hip
    if (S < 64 && L >= 8192 && !capture_open()) {
        size_t G = 256;
        if (outer > 1) while (G > 1 && L % G != 0) G /= 2;
        const size_t L0 = L / G * G, rem = L - L0;
        if (G >= 16 && G * S >= 256) {
            T* P = (T*)scratch(outer * (G + 1) * S * sizeof(T) + 256, 2);
            if (!P) return;
            wreduce<T, R>(in, P, outer, L0 / G, G * S, 0.0);
            if (rem) wreduce<T, R>(in + L0 * S, P + G * S, 1, rem, S, 0.0);
            wreduce<T, R>(P, out, outer, G + (rem ? 1 : 0), S, div);
            return;
        }
    }
    {
        // wide rows and a long axis: one 16-wave block per CU covers the memory latency, so few chunks (often none)
        constexpr size_t V = 16 / sizeof(T);
        if (S % V == 0 && S / V >= WAVE && L >= 256) {
            const size_t base = outer * cdiv(S / V, (size_t)WAVE);
            size_t nch = 1;
            if (base < 256) nch = std::min<size_t>(cdiv((size_t)256, base), L / 256);
            if (nch < 1) nch = 1;
            const size_t clen = cdiv(L, nch);
            nch = cdiv(L, clen);
            if (nch == 1) {
                if (wcol_split_stage<T, R>(in, out, outer, L, S, 1, L, div)) return;
            } else {
                T* part = (T*)scratch(outer * nch * S * sizeof(T) + 256);
                if (!part) return;
                if (wcol_split_stage<T, R>(in, part, outer, L, S, (unsigned)nch, clen, 0.0)) {
                    wcol_stage<T, R>(part, out, outer, nch, S, 1, nch, div);
                    return;
                }
            }
        }
    }
    const size_t threads = outer * S / (S % (16 / sizeof(T)) == 0 ? 16 / sizeof(T) : 1);
    size_t chunks = 1;
    if (threads < 131072 && L >= 64) chunks = std::min<size_t>(cdiv((size_t)131072, threads), L / 32);
    const size_t chunk_len = cdiv(L, chunks);
    chunks = cdiv(L, chunk_len);
    if (chunks == 1) { wcol_stage<T, R>(in, out, outer, L, S, 1, L, div); return; }
    T* part = (T*)scratch(outer * chunks * S * sizeof(T) + 256);
    if (!part) return;
    if (!wcol_stage<T, R>(in, part, outer, L, S, (unsigned)chunks, chunk_len, 0.0)) return;
    wcol_stage<T, R>(part, out, outer, chunks, S, 1, chunks, div);
}

// sum/mean/max/min metadata: dims[n] | strides[n] | red_len[r] | red_stride[r] | offset
template <class T, class R>
static void wreduce_axis(size_t num_els, size_t num_dims, size_t nred, const size_t* md, const T* in, T* out, bool mean) {
    if (!md || !in || !out) { set_status(ERR_INVALID, "reduce: null argument"); return; }
    if (nred != 1) { set_status(ERR_UNSUPPORTED, "reduce: exactly one reduced dim is supported"); return; }
    if (num_els == 0) return;
    const size_t* dims = md;
    const size_t* strides = md + num_dims;
    const size_t L = md[2 * num_dims], s = md[2 * num_dims + 1], offset = md[2 * num_dims + 2];
    if (L == 0) { set_status(ERR_INVALID, "reduce: zero-length axis"); return; }
    const double div = mean ? (double)L : 0.0;
    const T* src = in + offset;
    const size_t out_size = num_els / L;
    if (out_size == 0) return;
    if (ref_is_contiguous(num_dims, dims, strides) && s != 0 && num_els % (L * s) == 0) {
        wreduce<T, R>(src, out, num_els / (L * s), L, s, div);
        return;
    }
    if (num_els >= (1ull << 31)) { set_status(ERR_TOO_LARGE, "reduce: strided input with 2^31 or more elements"); return; }
    // A large strided input whose logical index space divides into whole slices is copied into logical order (the
    // elementwise identity walks the view by the reference's index rule) and reduced as the contiguous layout
    // [outer, L, s] the reference's formula describes - see reduce_axis in reduce.hip.
    {
        const size_t se = s != 0 ? s : 1;
        if (num_els >= (1u << 18) && num_dims <= 64 && num_els % (L * se) == 0 && !capture_open()) {
            T* tmp = (T*)scratch(num_els * sizeof(T), 1);
            if (!tmp) return;
            size_t cs[64];
            contiguous_strides(num_dims, dims, cs);
            const size_t* ins[1] = {strides};
            const void* inp[1] = {src};
            ew_launch<OpIdentity<T>>(num_els, num_dims, dims, cs, ins, tmp, inp, OpIdentity<T>{});
            wreduce<T, R>(tmp, out, num_els / (L * se), L, se, div);
            return;
        }
    }
    if (num_dims > (size_t)MAXD) { set_status(ERR_UNSUPPORTED, "reduce: strided input of rank above 8"); return; }
    NdSpace<1> sp;            // not collapsed: the walk must visit the dims exactly as the reference's index function does
    sp.ndims = (int)(num_dims ? num_dims : 1);
    for (int d = 0; d < MAXD; ++d) {
        sp.dims[d] = d < (int)num_dims ? (uint32_t)dims[d] : 1;
        sp.div[d] = make_fastdiv(sp.dims[d]);
        sp.strides[0][d] = d < (int)num_dims ? (int64_t)strides[d] : 0;
    }
    hipLaunchKernelGGL((wgeneric_kernel<T, R>), dim3((unsigned)cdiv(out_size, (size_t)WB)), dim3(WB), 0, stream(), sp, src, out, num_els, out_size, L, s, div);
    MXH_LAUNCH_CHECK("reduce_wide_generic");
}

// `0 + x` of a sum_to_shape that reduces nothing (f64: -0 becomes +0)
template <class T> struct WZeroPlus {
    using In = T; using Out = T; static constexpr int NIN = 1;
    __device__ T operator()(T x) const { return WSum::op<T>((T)0, x); }
};

// sum_to_shape metadata: in_dims[n] | in_strides[n] | out_dims[n] | offset.  Contiguous inputs only for these dtypes:
// runs of kept and of reduced dims are merged and every reduced run is one [outer, L, S] reduction, last run first.
template <class T>
static void wsum_to_shape(size_t num_els, size_t num_dims, const size_t* md, const T* in, T* out) {
    if (!md || !in || !out) { set_status(ERR_INVALID, "sum_to_shape: null argument"); return; }
    if (num_els == 0) return;
    if (num_dims > 64) { set_status(ERR_INVALID, "sum_to_shape: rank above 64"); return; }
    const size_t* in_dims = md;
    const size_t* in_strides = md + num_dims;
    const size_t* out_dims = md + 2 * num_dims;
    const T* src = in + md[3 * num_dims];
    if (!ref_is_contiguous(num_dims, in_dims, in_strides)) { set_status(ERR_UNSUPPORTED, "sum_to_shape: strided input is not supported for this dtype"); return; }
    size_t g_len[64];
    bool g_red[64];
    int ng = 0, nred = 0;
    for (size_t d = 0; d < num_dims; ++d) {
        if (out_dims[d] == 0 || (out_dims[d] != 1 && out_dims[d] != in_dims[d])) { set_status(ERR_UNSUPPORTED, "sum_to_shape: output dim must be 1 or the input dim"); return; }
        if (in_dims[d] == 1) continue;
        const bool red = out_dims[d] == 1;
        if (ng > 0 && g_red[ng - 1] == red) g_len[ng - 1] *= in_dims[d];
        else { g_len[ng] = in_dims[d]; g_red[ng] = red; ++ng; }
    }
    for (int g = 0; g < ng; ++g) nred += g_red[g];
    if (nred == 0) { ew_unary(num_els, 1, nullptr, src, out, WZeroPlus<T>{}); return; }
    // temporaries: two halves of slot 1 of the library scratch (the stage drivers' partials use slot 0)
    size_t smallest = ~(size_t)0;
    for (int g = 0; g < ng; ++g) if (g_red[g]) smallest = std::min<size_t>(smallest, g_len[g]);
    const size_t stage_bytes = nred > 1 ? ((num_els / smallest) * sizeof(T) + 255) / 256 * 256 : 0;
    T *ping = nullptr, *pong = nullptr;
    if (stage_bytes) {
        char* p = (char*)scratch(2 * stage_bytes + 256, 1);
        if (!p) return;
        ping = (T*)p; pong = (T*)(p + stage_bytes);
    }
    const T* cur = src;
    int left = nred;
    for (int g = ng - 1; g >= 0; --g) {
        if (!g_red[g]) continue;
        size_t outer = 1, inner = 1;
        for (int k = 0; k < g; ++k) outer *= g_len[k];
        for (int k = g + 1; k < ng; ++k) inner *= g_red[k] ? 1 : g_len[k];      // later reduced runs are gone already
        T* dst = --left == 0 ? out : (cur == ping ? pong : ping);
        wreduce<T, WSum>(cur, dst, outer, g_len[g], inner, 0.0);
        cur = dst;
    }
}

}  // namespace mxh

using namespace mxh;

#define MXH_WREDUCE_FOR(T, SUF)                                                                                 \
    extern "C" void hip_sum_##SUF(size_t n, size_t nd, size_t nr, const size_t* md, const T* in, T* out) { MXH_API; \
        wreduce_axis<T, WSum>(n, nd, nr, md, in, out, false);                                                   \
    }                                                                                                           \
    extern "C" void hip_max_##SUF(size_t n, size_t nd, size_t nr, const size_t* md, const T* in, T* out) { MXH_API; \
        wreduce_axis<T, WMax>(n, nd, nr, md, in, out, false);                                                   \
    }                                                                                                           \
    extern "C" void hip_min_##SUF(size_t n, size_t nd, size_t nr, const size_t* md, const T* in, T* out) { MXH_API; \
        wreduce_axis<T, WMin>(n, nd, nr, md, in, out, false);                                                   \
    }                                                                                                           \
    extern "C" void hip_sum_to_shape_##SUF(size_t n, size_t nd, const size_t* md, const T* in, T* out) { MXH_API; \
        wsum_to_shape<T>(n, nd, md, in, out);                                                                   \
    }
MXH_WREDUCE_FOR(double, f64)
MXH_WREDUCE_FOR(uint8_t, u8)
MXH_WREDUCE_FOR(uint16_t, u16)
MXH_WREDUCE_FOR(uint32_t, u32)
MXH_WREDUCE_FOR(uint64_t, u64)
MXH_WREDUCE_FOR(int8_t, i8)
MXH_WREDUCE_FOR(int16_t, i16)
MXH_WREDUCE_FOR(int32_t, i32)
MXH_WREDUCE_FOR(int64_t, i64)
extern "C" void hip_mean_f64(size_t n, size_t nd, size_t nr, const size_t* md, const double* in, double* out) { MXH_API;
    wreduce_axis<double, WSum>(n, nd, nr, md, in, out, true);
}
