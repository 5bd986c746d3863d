// im2col / col2im.  Replace cuda_conv2d_im2col_<T> / cuda_conv2d_col2im_<T> of
// crates/maidenx_cuda/src/nn/conv.rs:12-24 with the CPU semantics of
// crates/maidenx_cpu/src/nn/conv.rs:13-149.
// Metadata (12 slots, as the kernel reads them): B, C, H, W, kh, kw, oh, ow, pad_h, pad_w,
// stride_h, stride_w.
//   im2col : col[b][(c*kh+i)*kw+j][ho*ow+wo] = in[b,c,ho*sh-ph+i, wo*sw-pw+j] or 0.  Write-bound.
//            Whole column matrix with ow a multiple of the vector width: a block stages the input
//            rows of one (b, c) plane (or a band of it) once in a zero-padded LDS tile and streams
//            the kh*kw shifted copies out as 128-bit stores, so no global-load latency sits in
//            front of a store.  Otherwise (truncated num_els, odd widths, tiles beyond LDS): one
//            thread per vector or element with the shifted reads served by cache.
//   col2im : gather form with the reference's fixed summation order (ho then wo ascending, at
//            most kh*kw terms), so the result is bit-exact and deterministic; column indices at
//            or beyond num_els are skipped exactly as the reference does.
#include "elementwise.hpp"
#include "mxh.hpp"

namespace mxh {

struct ConvMeta {
    uint32_t B, C, H, W, kh, kw, oh, ow, ph, pw, sh, sw;
    FastDiv d_owv, d_oh, d_kw, d_kh, d_C;      // im2col index walk
    FastDiv d_W, d_H, d_Cc, d_sh, d_sw;        // col2im index walk
};

constexpr int CB = 256;

template <class T, int VEC>
struct alignas(sizeof(T) * VEC) CVec { T v[VEC]; };

template <class T, int VEC>
__global__ __launch_bounds__(CB) void im2col_kernel(ConvMeta m, const T* __restrict__ in, T* __restrict__ col, size_t nvec,
                                                    size_t num_els) {
    size_t v = (size_t)blockIdx.x * CB + threadIdx.x;
    if (v >= nvec) return;
    uint32_t r = (uint32_t)v, wov, ho, j, i, c, b;
    fd_divmod(r, m.d_owv, r, wov);
    fd_divmod(r, m.d_oh, r, ho);
    fd_divmod(r, m.d_kw, r, j);
    fd_divmod(r, m.d_kh, r, i);
    fd_divmod(r, m.d_C, b, c);
    int hi = (int)(ho * m.sh) - (int)m.ph + (int)i;
    const T* src = in + ((size_t)(b * m.C + c) * m.H + (hi >= 0 ? hi : 0)) * m.W;
    bool hok = hi >= 0 && hi < (int)m.H;
    CVec<T, VEC> o;
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
        int wi = (int)((wov * VEC + e) * m.sw) - (int)m.pw + (int)j;
        bool ok = hok && wi >= 0 && wi < (int)m.W;
        o.v[e] = ok ? src[wi] : T{};
    }
    size_t base = v * VEC;
    if (base + VEC <= num_els) *(CVec<T, VEC>*)(col + base) = o;
    else
        for (int e = 0; e < VEC; ++e) if (base + e < num_els) col[base + e] = o.v[e];
}

// im2col through LDS: one block owns a band of output rows of one (b, c) plane.  The input rows the
// band needs are read once into a zero-padded LDS tile [HP][WP] (so the copy loop has no bounds
// checks and no global-load latency), then the kh*kw shifted copies leave as 16-byte stores.
struct BandMeta {
    uint32_t nb, bands, HP, WP, nvec_seg;       // output rows per band, bands per plane, tile extent, vectors per (i, j) segment
    uint32_t vec_in;                            // the input rows are whole aligned 16-byte vectors
    FastDiv d_WP, d_bands, d_seg, d_owv, d_kw, d_wv;
};

// STREAM: the column matrix will not fit the last-level cache, so its stores carry the non-temporal hint.
template <class T, int VEC, bool STREAM = false>
__global__ __launch_bounds__(CB) void im2col_band_kernel(ConvMeta m, BandMeta k, const T* __restrict__ in, T* __restrict__ col) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    T* tile = (T*)smem;
    uint32_t plane, band;
    fd_divmod(blockIdx.x, k.d_bands, plane, band);            // plane = b*C + c
    const uint32_t ho0 = band * k.nb;
    const uint32_t nrows = min(k.nb, m.oh - ho0);
    const int hi0 = (int)(ho0 * m.sh) - (int)m.ph;             // input row of tile row 0
    const uint32_t hp = (nrows - 1) * m.sh + m.kh;             // tile rows this band uses
    const T* src = in + (size_t)plane * m.H * m.W;
    if (k.vec_in) {
        // The band's input rows as 16-byte vectors, up to four a thread, all requested before anything else happens: one
        // memory latency for the tile.  (Element by element, each behind its own bounds test, a thread waited for fourteen
        // loads one after the other - and every block of the launch did so at the same time, the grid being one round of
        // blocks: a fifth of the kernel passed before the first store.)  The tile is zeroed while the loads are in flight.
        const uint32_t wv = m.W / VEC;
        const int r_lo = hi0 < 0 ? -hi0 : 0, r_hi = min((int)hp, (int)m.H - hi0);       // tile rows that exist in the input
        const uint32_t nload = r_hi > r_lo ? (uint32_t)(r_hi - r_lo) * wv : 0u;
        const T* first = src + (size_t)(hi0 + r_lo) * m.W;
        for (uint32_t base = 0; base < nload || base == 0; base += 4 * CB) {
            CVec<T, VEC> v[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t idx = base + q * CB + threadIdx.x;
                if (idx < nload) v[q] = *(const CVec<T, VEC>*)(first + (size_t)idx * VEC);
            }
            if (base == 0) {
                CVec<T, VEC> z;
#pragma unroll
                for (int e = 0; e < VEC; ++e) z.v[e] = T{};
                const uint32_t nz = (hp * k.WP * (uint32_t)sizeof(T) + 15) / 16;      // (the tile's allocation is a whole number of vectors)
                for (uint32_t i = threadIdx.x; i < nz; i += CB) ((CVec<T, VEC>*)tile)[i] = z;
                __syncthreads();
            }
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t idx = base + q * CB + threadIdx.x;
                if (idx < nload) {
                    uint32_t r, cv;
                    fd_divmod(idx, k.d_wv, r, cv);
                    T* t = tile + ((uint32_t)r_lo + r) * k.WP + m.pw + cv * VEC;
#pragma unroll
                    for (int e = 0; e < VEC; ++e) t[e] = v[q].v[e];
                }
            }
        }
    } else {
        for (uint32_t idx = threadIdx.x; idx < hp * k.WP; idx += CB) {
            uint32_t r, cidx;
            fd_divmod(idx, k.d_WP, r, cidx);
            int hi = hi0 + (int)r, wi = (int)cidx - (int)m.pw;
            bool ok = hi >= 0 && hi < (int)m.H && wi >= 0 && wi < (int)m.W;
            tile[idx] = ok ? src[(size_t)hi * m.W + wi] : T{};
        }
    }
    __syncthreads();
    const uint32_t seg = nrows * (m.ow / VEC);                 // vectors of one (i, j) segment in this band
    const uint32_t total = seg * m.kh * m.kw;
    T* dst_plane = col + ((size_t)plane * m.kh * m.kw * m.oh + ho0) * m.ow;
    // full bands: divide by the constant segment length; the last (short) band of a plane divides by its own
    const bool full = nrows == k.nb;
    for (uint32_t idx = threadIdx.x; idx < total; idx += CB) {
        uint32_t ij, q, r, wov, i, j;
        if (full) fd_divmod(idx, k.d_seg, ij, q);
        else { ij = idx / seg; q = idx - ij * seg; }
        fd_divmod(q, k.d_owv, r, wov);
        fd_divmod(ij, k.d_kw, i, j);
        const T* t = tile + (r * m.sh + i) * k.WP + wov * VEC * m.sw + j;
        CVec<T, VEC> o;
#pragma unroll
        for (int e = 0; e < VEC; ++e) o.v[e] = t[e * m.sw];
        st_vec<STREAM>((CVec<T, VEC>*)(dst_plane + ((size_t)ij * m.oh + r) * m.ow + wov * VEC), o);
    }
}

template <class T> __device__ inline T acc_add(T a, T b);
template <> __device__ inline float acc_add<float>(float a, float b) { return a + b; }
template <> __device__ inline double acc_add<double>(double a, double b) { return a + b; }
template <> __device__ inline bf16_t acc_add<bf16_t>(bf16_t a, bf16_t b) { return f2bf(bf2f(a) + bf2f(b)); }   // rounds per add
template <> __device__ inline f16_t acc_add<f16_t>(f16_t a, f16_t b) { return f2h(h2f(a) + h2f(b)); }

template <class T>
__global__ __launch_bounds__(CB) void col2im_kernel(ConvMeta m, const T* __restrict__ col, T* __restrict__ out, size_t n_out,
                                                    size_t num_els, bool accumulate) {
    // accumulate: out[idx] = out[idx] + (the sum), i.e. the in-place add of the result into a gradient that exists
    size_t idx = (size_t)blockIdx.x * CB + threadIdx.x;
    if (idx >= n_out) return;
    uint32_t r = (uint32_t)idx, w, h, c, b;
    fd_divmod(r, m.d_W, r, w);
    fd_divmod(r, m.d_H, r, h);
    fd_divmod(r, m.d_Cc, b, c);
    // every column index of this (b, c) plane is at least plane0; beyond num_els the reference skips them all
    // (the layer passes num_els = B*C*H*W, so most planes end here)
    const size_t plane0 = (size_t)(b * m.C + c) * m.kh * m.kw * m.oh * m.ow;
    if (plane0 >= num_els) { out[idx] = accumulate ? acc_add<T>(out[idx], T{}) : T{}; return; }
    uint32_t h_pad = h + m.ph, w_pad = w + m.pw;
    uint32_t hs = h_pad > m.kh - 1 ? h_pad - (m.kh - 1) : 0, ws = w_pad > m.kw - 1 ? w_pad - (m.kw - 1) : 0;
    uint32_t h_start, w_start, h_last, w_last, rem;
    fd_divmod(hs + m.sh - 1, m.d_sh, h_start, rem);
    fd_divmod(ws + m.sw - 1, m.d_sw, w_start, rem);
    fd_divmod(h_pad, m.d_sh, h_last, rem);
    fd_divmod(w_pad, m.d_sw, w_last, rem);
    uint32_t h_end = min(h_last + 1, m.oh), w_end = min(w_last + 1, m.ow);
    T sum = T{};
    for (uint32_t ho = h_start; ho < h_end; ++ho)
        for (uint32_t wo = w_start; wo < w_end; ++wo) {
            uint32_t i = h_pad - ho * m.sh, j = w_pad - wo * m.sw;
            if (i < m.kh && j < m.kw) {
                size_t ci = ((((size_t)(b * m.C + c) * m.kh * m.kw + i * m.kw + j) * m.oh + ho) * m.ow) + wo;
                if (ci < num_els) sum = acc_add<T>(sum, col[ci]);
            }
        }
    out[idx] = accumulate ? acc_add<T>(out[idx], sum) : sum;
}

// Unit stride along w: a thread owns VEC adjacent pixels of a row.  For a fixed tap (i, j) their column
// entries are adjacent too, so the column matrix streams in as (element-aligned) vectors; each pixel
// still adds its terms in the reference's order: ho ascending, then wo ascending, which is j descending.
template <class T, int N> struct alignas(sizeof(T)) CUVec { T v[N]; };

// KH, KW > 0: the kernel extent is known at compile time, so every tap's load is issued before the first
// add (the sums are latency-bound otherwise: one round trip per tap).  KH = KW = 0: run-time extent.
template <class T, int VEC, int KH, int KW>
__global__ __launch_bounds__(CB) void col2im_row_kernel(ConvMeta m, const T* __restrict__ col, T* __restrict__ out, size_t nvec,
                                                        size_t num_els, bool accumulate) {
    size_t idx = (size_t)blockIdx.x * CB + threadIdx.x;
    if (idx >= nvec) return;
    uint32_t r = (uint32_t)idx, wv, h, plane;
    fd_divmod(r, m.d_W, r, wv);            // d_W divides by W / VEC here
    fd_divmod(r, m.d_H, plane, h);
    T* dst = out + idx * VEC;
    CVec<T, VEC> acc, old;
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc.v[e] = old.v[e] = T{};
    if (accumulate) old = *(const CVec<T, VEC>*)dst;        // (requested before the taps: its latency passes with theirs)
    const size_t plane0 = (size_t)plane * m.kh * m.kw * m.oh * m.ow;
    if (plane0 < num_els) {
        const uint32_t h_pad = h + m.ph;
        // one tap: fetch the VEC column entries of (i, j, ho) that exist, and say which do
        auto fetch = [&](uint32_t i, int j, uint32_t ho, CUVec<T, VEC>& v) -> uint32_t {
            const int wo0 = (int)(wv * VEC + m.pw) - j;
            const int64_t ci0 = (int64_t)(plane0 + ((size_t)(i * m.kw + j) * m.oh + ho) * m.ow) + wo0;
            if (wo0 >= 0 && wo0 + VEC <= (int)m.ow && (size_t)ci0 + VEC <= num_els) {
                v = *(const CUVec<T, VEC>*)(col + ci0);
                return (1u << VEC) - 1;
            }
            uint32_t mask = 0;
#pragma unroll
            for (int e = 0; e < VEC; ++e) {
                const int wo = wo0 + e;
                const bool ok = wo >= 0 && wo < (int)m.ow && (size_t)(ci0 + e) < num_els;
                v.v[e] = ok ? col[ci0 + e] : T{};
                mask |= (uint32_t)ok << e;
            }
            return mask;
        };
        if constexpr (KH > 0) {
            CUVec<T, VEC> v[KH * KW];
            uint32_t mask[KH * KW];
            // ho ascending is i descending: ho = (h_pad - i) / sh where that division is exact
#pragma unroll
            for (int a = 0; a < KH; ++a) {
                const int i = KH - 1 - a;
                uint32_t ho = 0, rem = 1;
                if (h_pad >= (uint32_t)i) fd_divmod(h_pad - i, m.d_sh, ho, rem);
                const bool row_ok = rem == 0 && ho < m.oh;
#pragma unroll
                for (int c = 0; c < KW; ++c) {
                    mask[a * KW + c] = 0;
                    if (row_ok) mask[a * KW + c] = fetch(i, KW - 1 - c, ho, v[a * KW + c]);
                }
            }
#pragma unroll
            for (int k = 0; k < KH * KW; ++k)
#pragma unroll
                for (int e = 0; e < VEC; ++e)
                    if (mask[k] >> e & 1) acc.v[e] = acc_add<T>(acc.v[e], v[k].v[e]);
        } else {
            const uint32_t hs = h_pad > m.kh - 1 ? h_pad - (m.kh - 1) : 0;
            uint32_t h_start, h_last, rem;
            fd_divmod(hs + m.sh - 1, m.d_sh, h_start, rem);
            fd_divmod(h_pad, m.d_sh, h_last, rem);
            const uint32_t h_end = min(h_last + 1, m.oh);
            for (uint32_t ho = h_start; ho < h_end; ++ho) {
                const uint32_t i = h_pad - ho * m.sh;
                if (i >= m.kh) continue;
                for (int j = (int)m.kw - 1; j >= 0; --j) {
                    CUVec<T, VEC> v;
                    const uint32_t mask = fetch(i, j, ho, v);
#pragma unroll
                    for (int e = 0; e < VEC; ++e)
                        if (mask >> e & 1) acc.v[e] = acc_add<T>(acc.v[e], v.v[e]);
                }
            }
        }
    }
    if (accumulate) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc.v[e] = acc_add<T>(old.v[e], acc.v[e]);
    }
    *(CVec<T, VEC>*)dst = acc;
}

// need_stride: col2im divides by the stride slots (the reference panics on 0); im2col only multiplies by them
static bool parse_conv(const size_t* md, ConvMeta& m, bool need_stride) {
    for (int k = 0; k < 12; ++k) if (md[k] >= (1ull << 31)) return false;
    m.B = (uint32_t)md[0]; m.C = (uint32_t)md[1]; m.H = (uint32_t)md[2]; m.W = (uint32_t)md[3];
    m.kh = (uint32_t)md[4]; m.kw = (uint32_t)md[5]; m.oh = (uint32_t)md[6]; m.ow = (uint32_t)md[7];
    m.ph = (uint32_t)md[8]; m.pw = (uint32_t)md[9]; m.sh = (uint32_t)md[10]; m.sw = (uint32_t)md[11];
    return (!need_stride || (m.sh != 0 && m.sw != 0)) && m.kh != 0 && m.kw != 0;
}

template <class T>
void im2col(size_t num_els, const size_t* md, const T* in, T* col) {
    if (!md || !in || !col) return;    // the reference returns silently
    ConvMeta m;
    if (!parse_conv(md, m, false)) { set_status(ERR_INVALID, "im2col: bad metadata"); return; }
    size_t full = (size_t)m.B * m.C * m.kh * m.kw * m.oh * m.ow;
    if (full == 0 || num_els == 0) return;
    if (full >= (1ull << 32)) { set_status(ERR_TOO_LARGE, "im2col: 2^32 or more column elements"); return; }
    size_t n = num_els < full ? num_els : full;
    constexpr int VEC = 16 / sizeof(T);
    bool vec = m.ow % VEC == 0 && ((uintptr_t)col % 16) == 0;
    uint32_t owv = vec ? m.ow / VEC : m.ow;
    m.d_owv = make_fastdiv(owv); m.d_oh = make_fastdiv(m.oh); m.d_kw = make_fastdiv(m.kw);
    m.d_kh = make_fastdiv(m.kh); m.d_C = make_fastdiv(m.C);
    if (vec && n == full && VEC > 1) {
        // band kernel: whole column matrix, rows a multiple of the vector width
        BandMeta k;
        k.WP = (m.ow - 1) * m.sw + m.kw;
        auto tile_bytes = [&](uint32_t nb) { return ((size_t)((nb - 1) * m.sh + m.kh) * k.WP * sizeof(T) + 15) / 16 * 16; };
        constexpr size_t LDS_MAX = 32 * 1024;
        if (tile_bytes(1) <= LDS_MAX) {
            uint32_t nb = m.oh;
            while (nb > 1 && tile_bytes(nb) > LDS_MAX) nb = (nb + 1) / 2;
            // Several rounds of blocks, as long as a segment stays a few KB long: a block first loads its tile and then only
            // stores, and in a launch of one round every block is in the same phase at the same time.  [32,64,56,56] 3x3:
            // whole planes (2048 blocks, one round) 48.8 us, bands of 28 / 14 / 7 rows 49.5 / 45.9 / 48.0 us.
            while (nb > 1 && (size_t)m.B * m.C * cdiv(m.oh, nb) < 8192 && (size_t)(nb / 2) * m.ow * sizeof(T) >= 2048) nb = (nb + 1) / 2;
            k.nb = nb;
            k.bands = (uint32_t)cdiv(m.oh, nb);
            k.HP = (nb - 1) * m.sh + m.kh;
            k.nvec_seg = nb * (m.ow / VEC);
            k.d_WP = make_fastdiv(k.WP); k.d_bands = make_fastdiv(k.bands); k.d_seg = make_fastdiv(k.nvec_seg);
            k.d_owv = make_fastdiv(m.ow / VEC); k.d_kw = make_fastdiv(m.kw);
            // whole input rows as vectors: the padded tile must hold every input column (a pad narrower than the kernel
            // reaches always does, but the metadata is the caller's)
            k.vec_in = m.W % VEC == 0 && ((uintptr_t)in % 16) == 0 && m.pw + m.W <= k.WP ? 1u : 0u;
            k.d_wv = make_fastdiv(k.vec_in ? m.W / VEC : 1);
            size_t blocks = (size_t)m.B * m.C * k.bands;
            if (blocks < (1ull << 31)) {
                if (ew_stream_bytes() != 0 && full * sizeof(T) >= ew_stream_bytes())
                    hipLaunchKernelGGL((im2col_band_kernel<T, VEC, true>), dim3((unsigned)blocks), dim3(CB), tile_bytes(nb), stream(), m, k, in, col);
                else
                    hipLaunchKernelGGL((im2col_band_kernel<T, VEC>), dim3((unsigned)blocks), dim3(CB), tile_bytes(nb), stream(), m, k, in, col);
                MXH_LAUNCH_CHECK("im2col");
                return;
            }
        }
    }
    size_t nvec = vec ? (n + VEC - 1) / VEC : n;
    if (vec) hipLaunchKernelGGL((im2col_kernel<T, VEC>), dim3(cdiv(nvec, CB)), dim3(CB), 0, stream(), m, in, col, nvec, n);
    else hipLaunchKernelGGL((im2col_kernel<T, 1>), dim3(cdiv(nvec, CB)), dim3(CB), 0, stream(), m, in, col, nvec, n);
    MXH_LAUNCH_CHECK("im2col");
}

template <class T>
void col2im(size_t num_els, const size_t* md, const T* col, T* out, bool accumulate = false) {
    if (!md || !col || !out) return;
    ConvMeta m;
    if (!parse_conv(md, m, true)) { set_status(ERR_INVALID, "col2im: bad metadata (stride slot is 0)"); return; }
    size_t n_out = (size_t)m.B * m.C * m.H * m.W;
    if (n_out == 0) return;
    if (n_out >= (1ull << 32)) { set_status(ERR_TOO_LARGE, "col2im: 2^32 or more output elements"); return; }
    m.d_H = make_fastdiv(m.H); m.d_Cc = make_fastdiv(m.C);
    m.d_sh = make_fastdiv(m.sh); m.d_sw = make_fastdiv(m.sw);
    constexpr int VEC = 16 / sizeof(T);
    if (m.sw == 1 && m.W % VEC == 0 && ((uintptr_t)out % 16) == 0) {
        m.d_W = make_fastdiv(m.W / VEC);
        size_t nvec = n_out / VEC;
        auto kern = col2im_row_kernel<T, VEC, 0, 0>;
        if (m.kh == 3 && m.kw == 3) kern = col2im_row_kernel<T, VEC, 3, 3>;
        else if (m.kh == 1 && m.kw == 1) kern = col2im_row_kernel<T, VEC, 1, 1>;
        else if (m.kh == 5 && m.kw == 5 && sizeof(T) == 4) kern = col2im_row_kernel<T, VEC, 5, 5>;
        hipLaunchKernelGGL(kern, dim3(cdiv(nvec, CB)), dim3(CB), 0, stream(), m, col, out, nvec, num_els, accumulate);
        MXH_LAUNCH_CHECK("col2im");
        return;
    }
    m.d_W = make_fastdiv(m.W);
    hipLaunchKernelGGL(col2im_kernel<T>, dim3(cdiv(n_out, CB)), dim3(CB), 0, stream(), m, col, out, n_out, num_els, accumulate);
    MXH_LAUNCH_CHECK("col2im");
}

}  // namespace mxh

using namespace mxh;

#define MXH_CONV_FOR(T, SUF)                                                                               \
    extern "C" void hip_conv2d_im2col_##SUF(size_t num_els, const size_t* md, const T* in, T* col) { MXH_API; \
        im2col<T>(num_els, md, in, col);                                                                   \
    }                                                                                                      \
    extern "C" void hip_conv2d_col2im_##SUF(size_t num_els, const size_t* md, const T* col, T* out) { MXH_API; \
        col2im<T>(num_els, md, col, out);                                                                  \
    }

MXH_CONV_FOR(float, f32)
// col2im added into a gradient that already exists: grad[i] = grad[i] + (what hip_conv2d_col2im_f32 would write to i)
extern "C" void hip_conv2d_col2im_add_f32(size_t num_els, const size_t* md, const float* col, float* grad) { MXH_API;
    col2im<float>(num_els, md, col, grad, true);
}
MXH_CONV_FOR(bf16_t, bf16)
MXH_CONV_FOR(f16_t, f16)
MXH_CONV_FOR(double, f64)      // (crates/maidenx_cuda/src/nn/conv.rs:35)
