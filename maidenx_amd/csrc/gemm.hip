// Matmul forward and backward.  Replaces cuda_matmul_<T> / cuda_matmul_backward_<T> of
// crates/maidenx_cuda/src/ops/matmul.rs:12-29 with the CPU semantics of
// crates/maidenx_cpu/src/ops/matmul.rs (batch stride = strides[0], backward contiguous-only).
//
// Every product on this path is one strided batched GEMM
//     out[b,i,j] = Σ_r X[b·xb + i·xi + r·xr] · Y[b·yb + r·yr + j·yj]         (out contiguous)
//   forward : X = A (i=m, r=k)          Y = B   (r=k, j=n)
//   grad_a  : X = dC (i=m, r=n)         Y = B   (r=n → stride 1, j=k → stride N)
//   grad_b  : X = A  (i=k → stride 1, r=m → stride K)   Y = dC (r=m, j=n)
// so the two transposed backward products need no materialised transpose: the operand whose
// reduction index is strided is turned while it is staged into LDS.
//
// Large products run on MFMA (v_mfma_f32_16x16x32_bf16 / v_mfma_f32_32x32x2_f32), f32 accumulate, one
// rounding at the end for bf16: 256x256 output tiles on 8-wave blocks (two waves per SIMD keep the matrix
// pipe fed), 128x128 on 4-wave blocks for problems with few tiles, 256x64 for narrow outputs; products
// with few tiles and a long reduction are split over the reduction and folded in a fixed order.
// bf16 uses the 16x16x32 instruction: the kernel is power-limited on real data, and that shape does
// about 15 % more work per joule than 32x32x16 (both measured in an MFMA-only loop on random operands).
// Operands sit in LDS as [row][k] with the reduction index contiguous, so a lane fetches its whole
// fragment with one 128-bit ds_read.
// Small or skinny products (the MLP's [10000,3]x[3,1] and its [3,10000]x[10000,1] gradient) use
// a thread-per-output kernel (bit-exact with the reference: k ascending, unfused f32) or a
// wave-per-output dot kernel.

#include <cstring>
#include <type_traits>

#include "fuse.hpp"
#include "gemm_host.hpp"
#include "gemm_small.hpp"
#include "mxh.hpp"

namespace mxh {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

constexpr int TK_BYTES = 128;    // reduction extent of one staged tile, in bytes per row

template <class T, int N> struct alignas(sizeof(T) * N) GVec { T v[N]; };
// 16 bytes as a native vector: staged tiles and fragments stay in registers as whole dwordx4 values
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
template <class T> __device__ inline uint32_t elem_bits(T v);
template <> __device__ inline uint32_t elem_bits<float>(float v) { return __builtin_bit_cast(uint32_t, v); }
template <> __device__ inline uint32_t elem_bits<bf16_t>(bf16_t v) { return v.bits; }
template <> __device__ inline uint32_t elem_bits<f16_t>(f16_t v) { return v.bits; }
// pack VEC elements (given one by one) into 16 bytes
template <class T> struct Pack16;
template <> struct Pack16<float> {
    u32x4 r;
    __device__ void set(int e, float v) { uint32_t b = __builtin_bit_cast(uint32_t, v); r[e] = b; }
};
template <> struct Pack16<bf16_t> {
    u32x4 r = {0u, 0u, 0u, 0u};
    __device__ void set(int e, bf16_t v) { r[e / 2] |= (uint32_t)v.bits << (16 * (e & 1)); }
};
template <> struct Pack16<f16_t> {
    u32x4 r = {0u, 0u, 0u, 0u};
    __device__ void set(int e, f16_t v) { r[e / 2] |= (uint32_t)v.bits << (16 * (e & 1)); }
};

// ---- staging one ROWS x TK operand tile into LDS as [row][TK + PAD] ---------------------------------
// `row` is the operand's output index (i for X, j for Y).  RCONT: the reduction index has stride 1
// in memory (natural); otherwise the row index has stride 1 and the tile is turned on the way in.
// load() only issues global loads into registers; store() does any re-packing and writes LDS, so the
// loads stay in flight across a whole k-tile of MFMAs.  NT = threads per block.
// Bank conflicts of the fragment reads (ds_read_b128; LDS serves such a read in four passes, and timing
// of access patterns says a pass takes lanes 0-7 with 24-31, 8-15 with 16-23, and the same in the upper
// half):
//   * 32x32 fragments (lane = row % 32, 16-byte chunk lane / 32): rows 16 bytes longer than the tile
//     (PITCH = TK + VEC) are conflict free;
//   * 16x16 fragments (lane = row % 16, chunk lane / 16): that padding leaves every read two-way
//     conflicted (9 instead of 4.5 cycles).  SWZ stores unpadded rows of 8 chunks with the chunk index
//     xor-ed by bits 1..3 of the row: both row sets of a pass then cover all 64 banks exactly once, and a
//     pair of rows (2q, 2q+1) shares its key, which is what the turned 16-bit staging writes together.
template <class T, bool RCONT, int ROWS, int NT, bool SWZ = false>
struct Stager {
    static constexpr int VEC = Elem<T>::VEC;
    static constexpr int TK = TK_BYTES / sizeof(T);
    static constexpr int PITCH = SWZ ? TK : TK + VEC;      // +16 bytes: keeps alignment, spreads banks
    static_assert(!SWZ || TK / VEC == 8, "the swizzle permutes 8 chunks per row");
    // element offset of 16-byte chunk `chunk` of row `row` inside a staged tile
    static __device__ __forceinline__ int at(int row, int chunk) {
        if constexpr (SWZ) chunk ^= (row >> 1) & 7;
        return row * PITCH + chunk * VEC;
    }
    static constexpr int NV = ROWS * TK / VEC / NT;        // 16-byte units per thread
    static constexpr bool PAIRS = !RCONT && sizeof(T) == 2;
    static_assert(NV >= 1 && (!PAIRS || NV % 2 == 0), "tile too small for this block size");
    u32x4 reg[NV];     // natural / 32-bit turned: final vectors.  16-bit turned: raw dwords (row pairs)

    // Buffer descriptor of one tile: the (uniform) tile origin is the base, so every lane addresses with
    // one loop-invariant 32-bit offset plus a scalar offset per load instead of a 64-bit pointer each.
    static __device__ __amdgpu_buffer_rsrc_t tile_rsrc(const T* base, int64_t s_row, int64_t s_red, uint32_t row0, uint32_t red0,
                                                       int records = 0x7fffffff) {
        const T* origin = base + (int64_t)row0 * s_row + (int64_t)red0 * s_red;
        return __builtin_amdgcn_make_buffer_rsrc((void*)origin, 0, records, 0x00020000);
    }
    // FAST: the tile lies fully inside the operand, wide accesses are aligned and offsets inside a tile
    // fit 31 bits (no checks at all)
    // A "unit" is what one pass of all threads loads: NU of them make the tile.  load()/store() take a
    // unit range so that a tile's traffic can be spread over the k-steps of the previous tile.
    static constexpr int NU = PAIRS ? NV / 2 : NV;
    // BOUND (with FAST): the tile's last rows may lie past the operand's nrows rows while its reduction range is whole.
    // The descriptor then ends with the operand's last element (row nrows - 1, reduction step nred - 1), and the
    // hardware returns zeros for every load past it.  A load of a row that does not exist either lies past that end or
    // reads other entries of the operand; what it brings only reaches outputs that are not stored.
    template <bool FAST, bool BOUND = false>
    __device__ void load(const T* __restrict__ base, int64_t s_row, int64_t s_red, uint32_t row0, uint32_t red0,
                         uint32_t nrows, uint32_t nred, int u0 = 0, int u1 = NU) {
        constexpr bool fast = FAST;
        static_assert(!BOUND || FAST, "bounded loads: the unchecked form");
        const int t = threadIdx.x;
        int records = 0x7fffffff;
        if constexpr (BOUND) {
            // bytes from the tile's origin to the end of the operand, to a whole dword (the 16-bit row pairs are loaded as
            // dwords; the operand starts on a dword and its strides are even, so its last dword is its own memory)
            const int64_t last = (int64_t)(nrows - 1 - row0) * (RCONT ? s_row : 1) + (int64_t)(nred - 1 - red0) * (RCONT ? 1 : s_red);
            const int64_t left = ((last + 1) * (int64_t)sizeof(T) + 3) & ~(int64_t)3;
            records = nrows > row0 && nred > red0 ? (int)(left < 0x7fffffff ? left : 0x7fffffff) : 0;
        }
        if constexpr (RCONT) {
            constexpr int KV = TK / VEC;   // vectors per row
#pragma unroll
            for (int u = 0; u < NV; ++u) {
                if (u < u0 || u >= u1) continue;
                int id = t + u * NT;
                uint32_t row = row0 + id / KV, red = red0 + (id % KV) * VEC;
                const T* p = base + (int64_t)row * s_row + red;
                if constexpr (fast) {
                    uint32_t voff = (uint32_t)(((t / KV) * s_row + (t % KV) * VEC) * (int64_t)sizeof(T));
                    uint32_t soff = (uint32_t)((int64_t)u * (NT / KV) * s_row * (int64_t)sizeof(T));
                    // (bounded: the whole offset in the vector operand, which is what the range check is sure to see)
                    if constexpr (BOUND) reg[u] = __builtin_amdgcn_raw_buffer_load_b128(tile_rsrc(base, s_row, s_red, row0, red0, records), voff + soff, 0, 0);
                    else reg[u] = __builtin_amdgcn_raw_buffer_load_b128(tile_rsrc(base, s_row, s_red, row0, red0), voff, soff, 0);
                } else {
                    Pack16<T> pk;
#pragma unroll
                    for (int e = 0; e < VEC; ++e) pk.set(e, (row < nrows && red + e < nred) ? p[e] : Elem<T>::zero());
                    reg[u] = pk.r;
                }
            }
        } else if constexpr (PAIRS) {
            // 16-bit elements: lanes run along pairs of rows (one dword = rows 2q, 2q+1 at one reduction
            // step, 256 contiguous bytes per wave).  A unit gathers 8 steps = 8 dwords = reg[2u], reg[2u+1].
            constexpr int NP = ROWS / 2;
#pragma unroll
            for (int u = 0; u < NV / 2; ++u) {
                if (u < u0 || u >= u1) continue;
                int id = t + u * NT;
                uint32_t row = row0 + (id % NP) * 2, red = red0 + (id / NP) * VEC;
                const T* p = base + (int64_t)row + (int64_t)red * s_red;
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    uint32_t d;
                    if constexpr (fast) {
                        uint32_t voff = (uint32_t)(((t % NP) * 2 + (t / NP) * VEC * s_red) * (int64_t)sizeof(T));
                        uint32_t soff = (uint32_t)(((int64_t)u * (NT / NP) * VEC + e) * s_red * (int64_t)sizeof(T));
                        if constexpr (BOUND) d = __builtin_amdgcn_raw_buffer_load_b32(tile_rsrc(base, 1, s_red, row0, red0, records), voff + soff, 0, 0);
                        else d = __builtin_amdgcn_raw_buffer_load_b32(tile_rsrc(base, 1, s_red, row0, red0), voff, soff, 0);
                    } else {
                        uint32_t lo = (row < nrows && red + e < nred) ? p[(int64_t)e * s_red].bits : 0u;
                        uint32_t hi = (row + 1 < nrows && red + e < nred) ? p[(int64_t)e * s_red + 1].bits : 0u;
                        d = lo | (hi << 16);
                    }
                    reg[2 * u + e / 4][e % 4] = d;
                }
            }
        } else {
            // 32-bit elements: lanes run along the row index (stride 1 in memory); each unit gathers VEC
            // reduction steps of one row so that the LDS write is again one [row][k..k+VEC) vector.
#pragma unroll
            for (int u = 0; u < NV; ++u) {
                if (u < u0 || u >= u1) continue;
                int id = t + u * NT;
                uint32_t row = row0 + id % ROWS, red = red0 + (id / ROWS) * VEC;
                const T* p = base + (int64_t)row + (int64_t)red * s_red;
                Pack16<T> pk;
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    if constexpr (fast) {
                        uint32_t voff = (uint32_t)(((t % ROWS) + (t / ROWS) * VEC * s_red) * (int64_t)sizeof(T));
                        uint32_t soff = (uint32_t)(((int64_t)u * (NT / ROWS) * VEC + e) * s_red * (int64_t)sizeof(T));
                        if constexpr (BOUND) pk.r[e] = __builtin_amdgcn_raw_buffer_load_b32(tile_rsrc(base, 1, s_red, row0, red0, records), voff + soff, 0, 0);
                        else pk.r[e] = __builtin_amdgcn_raw_buffer_load_b32(tile_rsrc(base, 1, s_red, row0, red0), voff, soff, 0);
                    } else {
                        pk.set(e, (row < nrows && red + e < nred) ? p[(int64_t)e * s_red] : Elem<T>::zero());
                    }
                }
                reg[u] = pk.r;
            }
        }
    }
    __device__ void store(T* lds, int u0 = 0, int u1 = NU) const {
        const int t = threadIdx.x;
        if constexpr (PAIRS) {
            constexpr int NP = ROWS / 2;
#pragma unroll
            for (int u = 0; u < NV / 2; ++u) {
                if (u < u0 || u >= u1) continue;
                int id = t + u * NT;
                int row = (id % NP) * 2, ck = id / NP;
                // d[e] = (row, k+e) | (row+1, k+e) << 16  →  [row][k..k+8) and [row+1][k..k+8)
                u32x4 lo, hi;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    uint32_t d0 = reg[2 * u + (2 * e) / 4][(2 * e) % 4], d1 = reg[2 * u + (2 * e + 1) / 4][(2 * e + 1) % 4];
                    // one byte permute each (as shifts and masks this is four vector-ALU instructions per pair, and on this
                    // chip vector-ALU time is not hidden behind the MFMAs)
                    lo[e] = __builtin_amdgcn_perm(d1, d0, 0x05040100u);      // d0.lo16 | d1.lo16 << 16
                    hi[e] = __builtin_amdgcn_perm(d1, d0, 0x07060302u);      // d0.hi16 | d1.hi16 << 16
                }
                *(u32x4*)(lds + at(row, ck)) = lo;
                *(u32x4*)(lds + at(row + 1, ck)) = hi;
            }
        } else {
#pragma unroll
            for (int u = 0; u < NV; ++u) {
                if (u < u0 || u >= u1) continue;
                int id = t + u * NT, row, ck;
                if constexpr (RCONT) { constexpr int KV = TK / VEC; row = id / KV; ck = id % KV; }
                else { row = id % ROWS; ck = id / ROWS; }
                *(u32x4*)(lds + at(row, ck)) = reg[u];
            }
        }
    }
};

// ---- the column matrix of a convolution as a left operand that is never stored -----------------------
// What conv2d_im2col writes for an input [B,C,H,W] is the buffer col[b][(c*kh+i)*kw+j][ho*ow+wo]; the Conv2d layer
// reads that buffer as a row-major matrix [B*oh*ow, C*kh*kw] (nn/layers/conv.rs:222, :279), i.e. entry (m, k) is flat
// index f = m*K + k of the buffer, whatever plane and pixel that happens to be.  Rows [b*P, (b+1)*P) of the matrix are
// batch b's part of the buffer (P = oh*ow), so within a batch the entry sits in plane (m - b*P)*K + k) / P at pixel
// (...) % P.  A staged tile of the matrix is gathered straight from the input (which the caches hold: it is a ninth of
// the matrix for a 3x3 kernel) instead of from a stored copy.
struct ColsView {
    const float* in;
    uint32_t K, P;                 // columns of the matrix (C*kh*kw), pixels of a plane (oh*ow)
    uint32_t H, W, HW, CHW, sh, sw;
    int32_t ph, pw;
    FastDiv d_P, d_khkw, d_kw, d_ow;
};
// The unit of the gather: matrix row m, columns k4 .. k4+3 (k4 a multiple of four).  VEC4: the four are neighbours in
// one output row (K and ow multiples of four), located once; otherwise one by one.  `live`: bit e = entry e is wanted.
template <bool VEC4>
__device__ __forceinline__ f32x4 cols_gather4(const ColsView& v, uint32_t m, uint32_t k4, uint32_t live) {
    f32x4 val = {0.0f, 0.0f, 0.0f, 0.0f};
    const uint32_t b = fd_div(m, v.d_P);
    const uint32_t f0 = (m - b * v.P) * v.K + k4;           // flat index inside batch b
    const float* plane0 = v.in + (size_t)b * v.CHW;
    auto locate = [&](uint32_t f, const float*& row, int32_t& wi) -> bool {      // the input row and column of flat index f
        uint32_t ckk, pix, ho, wo, c, t, i, j;
        fd_divmod(f, v.d_P, ckk, pix);
        fd_divmod(pix, v.d_ow, ho, wo);
        fd_divmod(ckk, v.d_khkw, c, t);
        fd_divmod(t, v.d_kw, i, j);
        const int32_t hi = (int32_t)(ho * v.sh + i) - v.ph;
        wi = (int32_t)(wo * v.sw + j) - v.pw;
        const bool ok = (uint32_t)hi < v.H;
        row = plane0 + c * v.HW + (ok ? (uint32_t)hi * v.W : 0u);
        return ok;
    };
    if constexpr (VEC4) {
        const float* row;
        int32_t wi;
        const bool hok = locate(f0, row, wi);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int32_t w = wi + e * (int32_t)v.sw;
            const bool ok = hok && (uint32_t)w < v.W && ((live >> e) & 1u);
            const float x = row[ok ? w : 0];
            val[e] = ok ? x : 0.0f;
        }
    } else {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if (!((live >> e) & 1u)) continue;
            const float* row;
            int32_t wi;
            const bool ok = locate(f0 + e, row, wi) && (uint32_t)wi < v.W;
            const float x = row[ok ? wi : 0];
            val[e] = ok ? x : 0.0f;
        }
    }
    return val;
}

// Stages a ROWS x TK tile of the matrix (TURNED: of its transpose, so the tile's rows are columns k of the matrix and
// its reduction runs over the rows m) into the LDS layout [row][TK + pad] of Stager<float, ...>.  Either way a thread
// gathers units of four consecutive k at one m (consecutive lanes take consecutive units along k: neighbouring
// pixels); TURNED then writes the four to four LDS rows instead of one 16-byte vector to one.
template <bool TURNED, bool VEC4, int ROWS, int NT>
struct ColsStager {
    static constexpr int TK = TK_BYTES / 4, PITCH = TK + 4;
    static constexpr int NV = ROWS * TK / 4 / NT, NU = NV;
    static constexpr int KV = (TURNED ? ROWS : TK) / 4;        // units along k
    static_assert(NV >= 1 && NT % KV == 0, "tile too small for this block size");
    f32x4 reg[NV];
    template <bool FAST>
    __device__ void load_cols(const ColsView& v, uint32_t row0, uint32_t red0, uint32_t nrows, uint32_t nred, int u0 = 0, int u1 = NU) {
        const int t = threadIdx.x;
#pragma unroll
        for (int u = 0; u < NV; ++u) {
            if (u < u0 || u >= u1) continue;
            const int id = t + u * NT;
            const uint32_t m = (TURNED ? red0 : row0) + id / KV, k4 = (TURNED ? row0 : red0) + (id % KV) * 4;
            uint32_t live = 0xFu;
            if constexpr (!FAST) {
                const uint32_t nm = TURNED ? nred : nrows, nk = TURNED ? nrows : nred;
                live = m >= nm || k4 >= nk ? 0u : nk - k4 >= 4 ? 0xFu : (1u << (nk - k4)) - 1u;
            }
            if (FAST || live) reg[u] = cols_gather4<VEC4>(v, m, k4, live);
            else reg[u] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        }
    }
    __device__ void store(float* lds, int u0 = 0, int u1 = NU) const {
        const int t = threadIdx.x;
#pragma unroll
        for (int u = 0; u < NV; ++u) {
            if (u < u0 || u >= u1) continue;
            const int id = t + u * NT;
            if constexpr (!TURNED) {
                *(f32x4*)(lds + (id / KV) * PITCH + (id % KV) * 4) = reg[u];
            } else {
                float* dst = lds + (id % KV) * 4 * PITCH + id / KV;
#pragma unroll
                for (int e = 0; e < 4; ++e) dst[e * PITCH] = reg[u][e];
            }
        }
    }
};

template <class T> struct Mma;
template <> struct Mma<bf16_t> {
    static __device__ void run(const u32x4& a, const u32x4& b, f32x16& c) {
        c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
    // 16x16 tiles, 32 reduction steps per instruction: lane (row l%16) holds k = 8*(l/16) .. +7
    static __device__ void run(const u32x4& a, const u32x4& b, f32x4& c) {
        c = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
};
template <> struct Mma<f16_t> {
    static __device__ void run(const u32x4& a, const u32x4& b, f32x16& c) {
        c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
    static __device__ void run(const u32x4& a, const u32x4& b, f32x4& c) {
        c = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
    }
};
template <> struct Mma<float> {
    // one 16-byte fragment feeds four 32x32x2 steps; lane (row, h) holds k = 4h .. 4h+3 of an
    // 8-wide slice, and step e pairs element e of both operands — any fixed pairing of k is valid.
    static __device__ void run(const u32x4& a, const u32x4& b, f32x16& c) {
        // (whole-vector casts: a bit cast applied to a single vector element reads element 0)
        const f32x4 af = __builtin_bit_cast(f32x4, a), bf = __builtin_bit_cast(f32x4, b);
#pragma unroll
        for (int e = 0; e < 4; ++e) c = __builtin_amdgcn_mfma_f32_32x32x2f32(af[e], bf[e], c, 0, 0, 0);
    }
};

// Block = WM x WN waves, each wave MI x MJ MFMA tiles of TS x TS: block tile (TS*MI*WM) x (TS*MJ*WN).
//   Big  : 4 x 2 waves of 2 x 4 tiles = 256 x 256, 512 threads.  One wave alone can issue a 32x32x16
//          MFMA only every other slot of the matrix pipe, so the pipe needs two waves per SIMD: 8 waves
//          per CU with 128 accumulator registers each (measured: 1.29 vs 1.81 PFLOP/s for an
//          MFMA-only loop with one vs two waves per SIMD).
//   Small: 2 x 2 waves of 2 x 2 tiles = 128 x 128, 256 threads, for problems with few tiles.
// The MFMA is issued with the operands swapped (Y fragment as "A"), so the accumulator of a lane
// holds 4 consecutive output columns of one output row and leaves as one packed store.
// TS = 16 (bf16 only): the same block and wave tiles built from 16x16x32 MFMAs.  On random data the
// matrix pipe sustains about 15 % more under the power limit with these than with 32x32x16 (an
// MFMA-only loop: 2.1 against 1.85 PFLOP/s; both reach 2.45 on constant data).
template <int WM_, int WN_, int MI_, int MJ_, int TS_ = 32> struct GemmCfg {
    static constexpr int WM = WM_, WN = WN_, MI = MI_, MJ = MJ_, TS = TS_;
    static constexpr int NT = WAVE * WM * WN, TM = TS * MI * WM, TN = TS * MJ * WN;
    using Acc = typename std::conditional<TS == 32, f32x16, f32x4>::type;
};
template <class T> struct Cfgs {
    using Big = GemmCfg<4, 2, 2, 4>;
    using Small = GemmCfg<2, 2, 2, 2>;
    using Tall = GemmCfg<2, 2, 1, 1>;     // 64 x 64, four blocks per CU: few output columns or a short reduction (see gemm_dispatch)
    using Flat = GemmCfg<1, 4, 1, 1>;     // 32 x 128: at most 32 output rows
};
template <> struct Cfgs<bf16_t> {
    using Big = GemmCfg<4, 2, 4, 8, 16>;
    using Small = GemmCfg<2, 2, 4, 4, 16>;
    using Tall = GemmCfg<2, 2, 2, 2, 16>;     // 64 x 64 (the conv-shaped bf16 weight gradient: 49 us, 205 us with 256 x 64 tiles)
    using Flat = Tall;                        // (a 32-row tile is too small for the turned 16-bit stager's row pairs)
};
template <> struct Cfgs<f16_t> : Cfgs<bf16_t> {};

// swapped operands: accumulator element e of tile (a, c) is output row i0 + .. + lane%32 and output
// column j0 + .. + 8*(e/4) + 4*(lane/32) + e%4  → four consecutive columns per group of 4 elements
// (16x16 tiles: one group of 4: column j0 + .. + 4*(lane/16) + e, row lane%16)
template <class O, class Cfg, bool FAST, bool EDGE = false>      // EDGE: FAST, but rows from g.I and columns from g.J on do not exist
__device__ __forceinline__ void store_tile(O* out, const typename Cfg::Acc (&acc)[Cfg::MI][Cfg::MJ], const GemmArgs& g, uint32_t i0, uint32_t j0,
                                           int wm, int wn, int lane) {
    constexpr int MI = Cfg::MI, MJ = Cfg::MJ, TS = Cfg::TS;
    const int lrow = lane % TS;
    const bool vec_store = FAST || ((g.J % 4 == 0) && ((uintptr_t)out % (4 * sizeof(O)) == 0));
#pragma unroll
    for (int a = 0; a < MI; ++a) {
        uint32_t row = i0 + wm * TS * MI + a * TS + lrow;
#pragma unroll
        for (int c = 0; c < MJ; ++c) {
#pragma unroll
            for (int q = 0; q < (TS == 32 ? 4 : 1); ++q) {
                uint32_t col = j0 + wn * TS * MJ + c * TS + (TS == 32 ? 8 * q + 4 * (lane / 32) : 4 * (lane / 16));
                if (!FAST && (row >= g.I || col >= g.J)) continue;
                if (EDGE && (row >= g.I || col >= g.J)) continue;      // (g.J is whole groups of four columns)
                O* dst = out + (int64_t)row * g.J + col;
                if (vec_store && (FAST || col + 4 <= g.J)) {
                    GVec<O, 4> v;
#pragma unroll
                    for (int e = 0; e < 4; ++e) v.v[e] = Elem<O>::st(acc[a][c][4 * q + e]);
                    *(GVec<O, 4>*)dst = v;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (col + e < g.J) dst[e] = Elem<O>::st(acc[a][c][4 * q + e]);
                }
            }
        }
    }
}

// The store of a Conv2d forward product: output row m = b * P + p of the [B*P, J] product is pixel p of batch b, and the
// layer wants out[b][j][p] = product[m][j] + bias[j] (nn/layers/conv.rs:222-232: reshape, two transposes, add).  A lane
// holds one row and 16 columns of a 32x32 tile, so for a given column the 32 lanes of a half-wave write 32 consecutive
// pixels: 128 contiguous bytes.  The addition is the elementwise kernel's f32 add on the same two values.
struct GemmEpi {
    const float* bias;
    uint32_t P;
    FastDiv d_P;
};
template <class Cfg>
__device__ __forceinline__ void store_tile_planes(float* out, const typename Cfg::Acc (&acc)[Cfg::MI][Cfg::MJ], const GemmArgs& g, const GemmEpi& e,
                                                  uint32_t i0, uint32_t j0, int wm, int wn, int lane) {
    constexpr int MI = Cfg::MI, MJ = Cfg::MJ, TS = Cfg::TS;
    static_assert(TS == 32, "f32 tiles");
#pragma unroll
    for (int a = 0; a < MI; ++a) {
        const uint32_t row = i0 + wm * TS * MI + a * TS + lane % TS;
        const uint32_t b = fd_div(row, e.d_P), p = row - b * e.P;
        float* plane0 = out + ((int64_t)b * g.J) * e.P + p;
#pragma unroll
        for (int c = 0; c < MJ; ++c)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t col = j0 + wn * TS * MJ + c * TS + 8 * q + 4 * (lane / 32);
                const f32x4 bias = *(const f32x4*)(e.bias + col);
#pragma unroll
                for (int k = 0; k < 4; ++k) plane0[(int64_t)(col + k) * e.P] = acc[a][c][4 * q + k] + bias[k];      // (never contracted: -ffp-contract=off)
            }
    }
}

// Folds the split-K partials in split order (deterministic) and rounds once.
template <class T>
__global__ __launch_bounds__(256) void gemm_fold_kernel(const float* __restrict__ part, T* __restrict__ out, size_t n, uint32_t splits) {
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    // sixteen partials in flight per thread (the launch is a few hundred blocks: taken one at a time, every partial
    // costs a memory latency); added in split order
    float acc = part[i];
    uint32_t s = 1;
    for (; s + 16 <= splits; s += 16) {
        float v[16];
#pragma unroll
        for (int k = 0; k < 16; ++k) v[k] = part[(size_t)(s + k) * n + i];
#pragma unroll
        for (int k = 0; k < 16; ++k) acc += v[k];
    }
    for (; s < splits; ++s) acc += part[(size_t)s * n + i];
    out[i] = Elem<T>::st(acc);
}

// Which tile, batch and reduction chunk a block works on.
struct TilePos {
    uint32_t ti, tj, b, split;
};
__device__ __forceinline__ TilePos tile_of_block(const GemmArgs& g) {
    // Blocks are handed to the 8 XCDs round robin, and each XCD has its own L2: give every XCD a compact
    // patch of the tile grid (GM tile rows x as many columns as it gets), so that the operand panels its
    // CUs stream are shared inside that L2 instead of being fetched by all eight.
    const uint32_t per = g.tiles_i * g.tiles_j;
    // Many small products (a batch of [512,1024] x [1024,1024]: eight tiles each): all tiles of one batch entry go to one
    // XCD, so that its operands are fetched once - handed out in launch order, the eight tiles of an entry land on eight
    // XCDs and every tile fetches both of its panels for itself (268 MB instead of 96 MB for that batch of 32).
    if (g.splits == 1 && g.batch % 8 == 0 && per <= 64) {
        const uint32_t xcd = blockIdx.x % 8, slot = blockIdx.x / 8;
        const uint32_t entry = slot / per, tile = slot - entry * per;
        TilePos t;
        t.ti = tile % g.tiles_i;
        t.tj = tile / g.tiles_i;
        t.b = entry * 8 + xcd;
        t.split = 0;
        return t;
    }
    uint32_t rest = blockIdx.x / per;
    uint32_t v = blockIdx.x - rest * per;
    if (per % 8 == 0) v = (v % 8) * (per / 8) + v / 8;
    constexpr uint32_t GM = 4;
    const uint32_t group = v / (GM * g.tiles_j), in_group = v - group * (GM * g.tiles_j);
    const uint32_t first_i = group * GM, rows = g.tiles_i - first_i < GM ? g.tiles_i - first_i : GM;
    TilePos t;
    t.ti = first_i + in_group % rows;
    t.tj = in_group / rows;
    t.b = rest % g.batch;
    t.split = rest / g.batch;
    return t;
}

// FAST: the tile lies inside the operands in all three extents and the wide accesses are aligned (no checks).
// PANEL: the block works through a run of consecutive output tiles (row-major over the tile grid: pos.ti is the first
// tile, pos.tj the number of tiles), one after the other, in the same pipeline: the k-tiles of the next output tile are
// requested while this one is being multiplied, and its stores leave while the next one works.  For products with a
// reduction of a few k-tiles only (a convolution's input gradient, [100352,64]x[64,576]): as one block per output tile
// such a product is 14112 short blocks, each of which pays the full memory latency for two k-tiles of work, and the four
// blocks a CU holds do not cover it.  The launch has as many blocks as the chip holds at once, with equal shares.
// XCOLS (f32): X is the column matrix of a convolution (XR) or its transpose (!XR), gathered from the input (ColsView);
// 2: four at a time (see cols_gather4), 1: one by one.
// RB: FAST for a tile whose last rows lie past g.I or whose last columns lie past g.J (the reduction whole k-tiles): X and Y
// are loaded through descriptors that end with their last entries, and the outputs that do not exist are not stored.
template <class T, bool XR, bool YR, class Cfg, bool FAST, bool PANEL = false, int XCOLS = 0, bool RB = false, bool PLANES = false>
__device__ __forceinline__ void gemm_mfma_body(const GemmArgs& g, const TilePos& pos, unsigned char* smem, const ColsView* cv = nullptr,
                                               const GemmEpi* epi = nullptr) {
    static_assert(!RB || (FAST && !PANEL && XCOLS == 0), "bounded rows: the unchecked body of stored operands");
    static_assert(!PLANES || (std::is_same<T, float>::value && FAST && !PANEL && !RB), "the Conv2d store: f32, whole tiles, no split");
    constexpr int TM = Cfg::TM, TN = Cfg::TN, MI = Cfg::MI, MJ = Cfg::MJ, NT = Cfg::NT;
    constexpr bool SWZ = Cfg::TS == 16;
    static_assert(!XCOLS || (std::is_same<T, float>::value && !PANEL), "the gathered operand is f32, one tile per block");
    using SX = typename std::conditional<XCOLS != 0, ColsStager<!XR, XCOLS == 2, TM, NT>, Stager<T, XR, TM, NT, SWZ>>::type;
    using SY = Stager<T, YR, TN, NT, SWZ>;
    constexpr int VEC = Elem<T>::VEC;
    constexpr int TK = SX::TK;
    constexpr int PITCH = SX::PITCH;
    T* lds_x = (T*)smem;                                  // [2][TM*PITCH]
    T* lds_y = lds_x + 2 * TM * PITCH;                    // [2][TN*PITCH]

    const uint32_t ti = pos.ti, tj = pos.tj, b = pos.b, split = pos.split;
    const uint32_t rb = split * g.r_chunk;                                  // this block reduces over [rb, re)
    const uint32_t re = g.R - rb < g.r_chunk ? g.R : rb + g.r_chunk;
    const uint32_t i0 = ti * TM, j0 = tj * TN;
    const T* X = (const T*)g.X + (int64_t)b * g.xb;
    const T* Y = (const T*)g.Y + (int64_t)b * g.yb;

    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
    const int wm = wave / Cfg::WN, wn = wave % Cfg::WN;
    constexpr int TS = Cfg::TS;
    const int lrow = lane % TS, lk = (lane / TS) * VEC;
    constexpr int KS = (WAVE / TS) * VEC;                   // reduction steps one MFMA (group) consumes


    // Software pipeline (all indices compile-time after unrolling, one barrier per k-tile).  While the
    // MFMAs work through LDS[cur] (tile kt), step s < S-1 of the tile
    //   * moves a share of the registers (tile kt+1, loaded one tile ago) into LDS[cur^1] and refills
    //     them with the same share of tile kt+2, so LDS writes and global loads trickle instead of burst,
    //   * reads the fragments of step s+1;
    // the last step starts with the barrier (LDS[cur^1] complete, LDS[cur] no longer read by anyone
    // once the fragments of step S-1 are in registers) and reads step 0 of the next tile under the cover
    // of its own MFMAs.  Loads past the last tile are redirected to it (harmless re-reads).
    // Steps per tile.  32x32 tiles: one per KS reduction steps, every step reads MI + MJ fragments and
    // issues MI*MJ MFMAs.  16x16 tiles: a k-step of 32 is cut in two halves of the column tiles, so a
    // step reads MJ/2 Y fragments (and the MI X fragments at the first half) and issues MI*MJ/2 MFMAs.
    constexpr int S = TS == 32 ? TK / KS : 2 * (TK / KS);
    constexpr int MJH = TS == 32 ? MJ : MJ / 2;
    static_assert(S >= 2 && S % 2 == 0, "fragment double buffer assumes an even number of steps");
    static_assert(TS == 32 || (sizeof(T) == 2 && MJ % 2 == 0), "16x16 tiles are for 16-bit operands");
    SX sx;
    SY sy;
    const uint32_t nk1 = (re - rb + TK - 1) / TK;                 // k-tiles of one output tile
    const uint32_t nk = PANEL ? nk1 * pos.tj : nk1;               // steps of the pipeline
    // where step q of the pipeline reads: its reduction offset and (PANEL) the first row and column of its output tile
    auto red_of = [&](uint32_t q) { return rb + (PANEL ? q % nk1 : q) * TK; };
    auto row_of = [&](uint32_t q) { return PANEL ? ((pos.ti + q / nk1) / g.tiles_j) * (uint32_t)TM : i0; };
    auto col_of = [&](uint32_t q) { return PANEL ? ((pos.ti + q / nk1) % g.tiles_j) * (uint32_t)TN : j0; };
    // units [u0, u1) of the X tile at (row, red) into the registers of stager st
    auto load_x = [&](SX& st, uint32_t row, uint32_t red, int u0, int u1) {
        if constexpr (XCOLS) st.template load_cols<FAST>(*cv, row, red, g.I, re, u0, u1);
        else st.template load<FAST, RB>(X, g.xi, g.xr, row, red, g.I, re, u0, u1);
    };
    {
        // tiles 0 and 1 are requested together (one memory latency instead of two); the accumulators are
        // not live yet, so the second set of staging registers costs nothing
        SX sx0;
        SY sy0;
        load_x(sx0, row_of(0), rb, 0, SX::NU);
        sy0.template load<FAST, RB>(Y, g.yj, g.yr, col_of(0), rb, g.J, re);
        const uint32_t q1 = nk > 1 ? 1u : 0u;
        load_x(sx, row_of(q1), red_of(q1), 0, SX::NU);
        sy.template load<FAST, RB>(Y, g.yj, g.yr, col_of(q1), red_of(q1), g.J, re);
        sx0.store(lds_x);
        sy0.store(lds_y);
    }
    __syncthreads();
    typename Cfg::Acc acc[MI][MJ];
#pragma unroll
    for (int a = 0; a < MI; ++a)
#pragma unroll
        for (int c = 0; c < MJ; ++c)
#pragma unroll
            for (int e = 0; e < (TS == 32 ? 16 : 4); ++e) acc[a][c][e] = 0.0f;

    const int frag_x = (wm * TS * MI + lrow) * PITCH + lk;   // + a*TS*PITCH + k-step*KS
    const int frag_y = (wn * TS * MJ + lrow) * PITCH + lk;
    // 16x16 tiles: the swizzled chunk of a lane differs per k-step, so one offset per step (the tile
    // offsets a * TS * PITCH keep bits 1..3 of the row and stay immediates)
    int frag_xk[2] = {0, 0}, frag_yk[2] = {0, 0};
    if constexpr (TS == 16) {
        static_assert(TS != 16 || TK / KS == 2, "two k-steps per staged tile");
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            frag_xk[ks] = SX::at(wm * TS * MI + lrow, lane / TS + ks * (KS / VEC));
            frag_yk[ks] = SY::at(wn * TS * MJ + lrow, lane / TS + ks * (KS / VEC));
        }
    }
    u32x4 fa[2][MI], fb[2][MJH];
    // fragments of step s from the tile at (bx, by)
    auto read_frags = [&](int s, const T* bx, const T* by) {
        if constexpr (TS == 32) {
#pragma unroll
            for (int a = 0; a < MI; ++a) fa[s & 1][a] = *(const u32x4*)(bx + frag_x + a * TS * PITCH + s * KS);
#pragma unroll
            for (int c = 0; c < MJ; ++c) fb[s & 1][c] = *(const u32x4*)(by + frag_y + c * TS * PITCH + s * KS);
        } else {
            const int ks = s >> 1, h = s & 1;
            if (h == 0) {
#pragma unroll
                for (int a = 0; a < MI; ++a) fa[ks & 1][a] = *(const u32x4*)(bx + frag_xk[ks] + a * TS * PITCH);
            }
#pragma unroll
            for (int c = 0; c < MJH; ++c) fb[s & 1][c] = *(const u32x4*)(by + frag_yk[ks] + (h * MJH + c) * TS * PITCH);
        }
    };
    auto mfmas = [&](int s) {
        if constexpr (TS == 32) {
#pragma unroll
            for (int a = 0; a < MI; ++a)
#pragma unroll
                for (int c = 0; c < MJ; ++c) Mma<T>::run(fb[s & 1][c], fa[s & 1][a], acc[a][c]);
        } else {
            const int ks = s >> 1, h = s & 1;
#pragma unroll
            for (int a = 0; a < MI; ++a)
#pragma unroll
                for (int c = 0; c < MJH; ++c) Mma<T>::run(fb[s & 1][c], fa[ks & 1][a], acc[a][h * MJH + c]);
        }
    };
    read_frags(0, lds_x, lds_y);

    for (uint32_t kt = 0; kt < nk; ++kt) {
        const int cur = kt & 1;
        const T* cx = lds_x + cur * TM * PITCH;
        const T* cy = lds_y + cur * TN * PITCH;
        T* nx = lds_x + (cur ^ 1) * TM * PITCH;
        T* ny = lds_y + (cur ^ 1) * TN * PITCH;
        const uint32_t qn = kt + 2 < nk ? kt + 2 : nk - 1;
        const uint32_t nt = red_of(qn), ni = row_of(qn), nj = col_of(qn);
#pragma unroll
        for (int s = 0; s < S; ++s) {
            if (s + 1 < S) {
                const int x0 = SX::NU * s / (S - 1), x1 = SX::NU * (s + 1) / (S - 1);
                const int y0 = SY::NU * s / (S - 1), y1 = SY::NU * (s + 1) / (S - 1);
                sx.store(nx, x0, x1);
                sy.store(ny, y0, y1);
                load_x(sx, ni, nt, x0, x1);
                sy.template load<FAST, RB>(Y, g.yj, g.yr, nj, nt, g.J, re, y0, y1);
                read_frags(s + 1, cx, cy);
            } else {
                __syncthreads();
                read_frags(0, nx, ny);
            }
            // keep the memory operations of the next stage ahead of this step's MFMAs: the matrix
            // pipe then works through them while LDS and the vector memory unit serve the next step
            mfmas(s);
#pragma unroll
            for (int i = 0; i < MI * MJH; ++i) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // one MFMA
                __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);   // one LDS write
                __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);   // one global load
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // one LDS read
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (PANEL) {
            if ((kt + 1) % nk1 == 0) {       // the last k-tile of an output tile: out it goes, and the accumulators start over
                store_tile<T, Cfg, FAST, RB>((T*)g.out, acc, g, row_of(kt), col_of(kt), wm, wn, lane);
#pragma unroll
                for (int a = 0; a < MI; ++a)
#pragma unroll
                    for (int c = 0; c < MJ; ++c)
#pragma unroll
                        for (int e = 0; e < (TS == 32 ? 16 : 4); ++e) acc[a][c][e] = 0.0f;
            }
        }
    }
    if constexpr (PANEL) return;

    if (g.splits > 1) {
        float* part = g.part + ((int64_t)split * g.batch + b) * g.I * g.J;
        store_tile<float, Cfg, FAST, RB>(part, acc, g, i0, j0, wm, wn, lane);
    } else if constexpr (PLANES) {
        store_tile_planes<Cfg>((float*)g.out, acc, g, *epi, i0, j0, wm, wn, lane);
    } else {
        store_tile<T, Cfg, FAST, RB>((T*)g.out + (int64_t)b * g.I * g.J, acc, g, i0, j0, wm, wn, lane);
    }
}

// ALIGNED: the operands allow the unchecked body wherever a whole tile lies inside them (the host has checked
// alignment, strides and that the reduction is a whole number of k-tiles); blocks on a ragged edge, and every block
// of an unaligned problem, take the checked body.
// whole tiles everywhere, one batch, no split: block b takes the tiles [b * per, (b + 1) * per) of the row-major tile grid
template <class T, bool XR, bool YR, class Cfg>
__global__ __launch_bounds__(Cfg::NT) void gemm_mfma_panel_kernel(GemmArgs g, uint32_t per) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const uint32_t tiles = g.tiles_i * g.tiles_j, first = blockIdx.x * per;
    if (first >= tiles) return;
    TilePos pos;
    pos.ti = first;
    pos.tj = tiles - first < per ? tiles - first : per;
    pos.b = 0;
    pos.split = 0;
    gemm_mfma_body<T, XR, YR, Cfg, true, true>(g, pos, smem);
}

// whole tiles everywhere, one batch, no split, both operands reduction-contiguous: the Conv2d forward product with its
// bias add and layout change in the store (GemmEpi)
template <class Cfg>
__global__ __launch_bounds__(Cfg::NT) void gemm_mfma_planes_kernel(GemmArgs g, GemmEpi e) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const TilePos pos = tile_of_block(g);
    gemm_mfma_body<float, true, true, Cfg, true, false, 0, false, true>(g, pos, smem, nullptr, &e);
}

template <class T, bool XR, bool YR, class Cfg, bool ALIGNED>
__global__ __launch_bounds__(Cfg::NT) void gemm_mfma_kernel(GemmArgs g) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const TilePos pos = tile_of_block(g);
    if constexpr (ALIGNED) {
        if ((pos.ti + 1) * Cfg::TM <= g.I && (pos.tj + 1) * Cfg::TN <= g.J) {
            gemm_mfma_body<T, XR, YR, Cfg, true>(g, pos, smem);
            return;
        }
        // A tile that runs past g.I or g.J.  (Not in the 256 x 256 configuration with both operands turned: it has no
        // register to spare, and with this body beside the other the compiler spills in it.)
        if constexpr (!(Cfg::TM >= 256 && !XR && !YR)) {
            gemm_mfma_body<T, XR, YR, Cfg, true, false, 0, true>(g, pos, smem);
            return;
        }
    }
    gemm_mfma_body<T, XR, YR, Cfg, false>(g, pos, smem);
}

template <bool XR, bool YR, class Cfg, bool ALIGNED, bool VEC4>
__global__ __launch_bounds__(Cfg::NT) void gemm_mfma_cols_kernel(GemmArgs g, ColsView v) {
    extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
    const TilePos pos = tile_of_block(g);
    if constexpr (ALIGNED) {
        if ((pos.ti + 1) * Cfg::TM <= g.I && (pos.tj + 1) * Cfg::TN <= g.J) {
            gemm_mfma_body<float, XR, YR, Cfg, true, false, VEC4 ? 2 : 1>(g, pos, smem, &v);
            return;
        }
    }
    gemm_mfma_body<float, XR, YR, Cfg, false, false, VEC4 ? 2 : 1>(g, pos, smem, &v);
}

// cv: X is the gathered column matrix of a convolution (f32), see ColsView
// r_split: the reduction length that decides how the reduction is cut (g.R is that length padded to whole k-tiles), 0: g.R
template <class T, bool XR, bool YR, class Cfg, bool FAST, int XCOLS = 0>
void launch_mfma_impl(GemmArgs g, const ColsView* cv = nullptr, uint32_t r_split = 0) {
    using SX = Stager<T, XR, Cfg::TM, Cfg::NT, Cfg::TS == 16>;
    constexpr size_t lds_bytes = (size_t)2 * (Cfg::TM + Cfg::TN) * SX::PITCH * sizeof(T);
    constexpr uint32_t TK = TK_BYTES / sizeof(T);
    g.tiles_i = cdiv(g.I, Cfg::TM);
    g.tiles_j = cdiv(g.J, Cfg::TN);
    size_t tiles = (size_t)g.tiles_i * g.tiles_j * g.batch;
    // Few output tiles and a long reduction (dB of a wide batch, the weight gradient of a convolution):
    // when the tiles cover less than half of the CUs, cut the reduction so that every CU has work,
    // each block keeping at least 8 k-tiles.
    g.splits = 1;
    g.r_chunk = g.R;
    g.part = nullptr;
    const size_t want_blocks = Cfg::NT >= 512 ? 256 : 512;       // one or two resident blocks per CU
    const uint32_t Rs = r_split ? r_split : g.R;
    if (tiles <= 128 && Rs >= 16 * TK) {
        uint32_t want = (uint32_t)std::min<size_t>(cdiv(want_blocks, tiles), Rs / (8 * TK));
        if (want > 1) {
            g.r_chunk = (uint32_t)(cdiv(cdiv(Rs, want), TK) * TK);
            g.splits = (uint32_t)cdiv(Rs, g.r_chunk);
        }
    }
    size_t blocks = tiles * g.splits;
    if (blocks >= (1ull << 31)) { set_status(ERR_TOO_LARGE, "matmul: too many tiles"); return; }
    const size_t n_out = (size_t)g.batch * g.I * g.J;
    if (g.splits > 1) {
        g.part = (float*)scratch(n_out * g.splits * sizeof(float));
        if (!g.part) return;
    }
    if constexpr (XCOLS != 0) {
        {
            auto ck = gemm_mfma_cols_kernel<XR, YR, Cfg, FAST, XCOLS == 2>;
            if (lds_bytes > (64u << 10)) {
                static bool allowed[64] = {false};     // per instantiation, indexed by device
                int dev = 0;
                MXH_HIP(hipGetDevice(&dev));
                if (dev < 0 || dev >= 64 || !allowed[dev]) {
                    MXH_HIP(hipFuncSetAttribute((const void*)ck, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
                    if (dev >= 0 && dev < 64) allowed[dev] = true;
                }
            }
            hipLaunchKernelGGL(ck, dim3((unsigned)blocks), dim3(Cfg::NT), lds_bytes, stream(), g, *cv);
            MXH_LAUNCH_CHECK("gemm_mfma_cols");
            if (g.splits > 1) {
                hipLaunchKernelGGL(gemm_fold_kernel<T>, dim3((unsigned)cdiv(n_out, 256)), dim3(256), 0, stream(), g.part, (T*)g.out, n_out, g.splits);
                MXH_LAUNCH_CHECK("gemm_fold");
            }
            return;
        }
    }
    if constexpr (FAST && std::is_same<Cfg, typename Cfgs<T>::Tall>::value) {
        // a reduction of a few k-tiles, many whole tiles: as many blocks as the chip holds, each with a run of tiles (see PANEL)
        constexpr size_t slots = 256 * 4;       // four blocks of this configuration fit a CU's LDS
        if (g.splits == 1 && g.batch == 1 && g.R <= 4 * TK && g.I % Cfg::TM == 0 && g.J % Cfg::TN == 0 && tiles >= 4 * slots && tiles < (1ull << 31)) {
            auto pk = gemm_mfma_panel_kernel<T, XR, YR, Cfg>;
            const uint32_t per = (uint32_t)cdiv(tiles, slots);
            hipLaunchKernelGGL(pk, dim3((unsigned)cdiv(tiles, (size_t)per)), dim3(Cfg::NT), lds_bytes, stream(), g, per);
            MXH_LAUNCH_CHECK("gemm_mfma_panel");
            return;
        }
    }
    auto kern = gemm_mfma_kernel<T, XR, YR, Cfg, FAST>;
    // more than 64 KB of LDS has to be allowed once per kernel and device (setting it twice is harmless)
    static bool attr_done[64] = {false};     // per instantiation, indexed by device
    int dev = 0;
    MXH_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= 64 || !attr_done[dev]) {
        MXH_HIP(hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
        if (dev >= 0 && dev < 64) attr_done[dev] = true;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)blocks), dim3(Cfg::NT), lds_bytes, stream(), g);
    MXH_LAUNCH_CHECK("gemm_mfma");
    if (g.splits > 1) {
        hipLaunchKernelGGL(gemm_fold_kernel<T>, dim3((unsigned)cdiv(n_out, 256)), dim3(256), 0, stream(), g.part, (T*)g.out, n_out, g.splits);
        MXH_LAUNCH_CHECK("gemm_fold");
    }
}

// One operand (nrows rows of R reduction steps, any strides) copied into the layout the unchecked body wants, in its own
// orientation: rows of Rp >= R steps each when the reduction index is the contiguous one (RCONT), else Rp rows of
// `pitch` entries.  Steps from R on and the entries past nrows are zeros.  One thread per entry of the copy.
template <class T, bool RCONT>
__global__ __launch_bounds__(256) void gemm_repack_kernel(const T* __restrict__ src, T* __restrict__ dst, uint32_t nrows, uint32_t R,
                                                          uint32_t Rp, uint32_t pitch, int64_t s_batch, int64_t s_row, int64_t s_red) {
    const uint32_t per = RCONT ? nrows * Rp : Rp * pitch;
    const uint32_t id = blockIdx.x * 256 + threadIdx.x;
    if (id >= per) return;
    const uint32_t b = blockIdx.y;
    const uint32_t row = RCONT ? id / Rp : id % pitch, red = RCONT ? id % Rp : id / pitch;
    T v = Elem<T>::zero();
    if (row < nrows && red < R) v = src[(int64_t)b * s_batch + (int64_t)row * s_row + (int64_t)red * s_red];
    dst[(size_t)b * per + id] = v;
}

// The unchecked kernel needs whole tiles in all three extents, 16-byte aligned rows for naturally laid
// out operands (4-byte aligned row pairs for turned 16-bit ones) and an output it can store 4 wide.
template <class T, bool XR, bool YR, class Cfg>
void launch_mfma(GemmArgs g) {
    constexpr int VEC = Elem<T>::VEC, TK = TK_BYTES / sizeof(T);
    auto op_ok = [&](const void* p, int64_t s_batch, int64_t s_row, int64_t s_red, bool rcont) {
        if (g.batch == 1) s_batch = 0;      // never applied
        if (rcont) return (uintptr_t)p % 16 == 0 && s_row % VEC == 0 && s_batch % VEC == 0;
        if (sizeof(T) == 2) return (uintptr_t)p % 4 == 0 && s_red % 2 == 0 && s_batch % 2 == 0;
        return true;
    };
    // per-thread offsets inside one tile are 32-bit
    auto span_ok = [&](int64_t s_row, int64_t s_red, int rows) {
        return s_row >= 0 && s_red >= 0 && ((int64_t)rows * s_row + (int64_t)TK * s_red) * (int64_t)sizeof(T) < (1ll << 31);
    };
    // (ragged tiles are decided per block inside the kernel)
    const bool x_fast = span_ok(g.xi, g.xr, Cfg::TM) && g.R % TK == 0 && op_ok(g.X, g.xb, g.xi, g.xr, XR);
    const bool y_fast = span_ok(g.yj, g.yr, Cfg::TN) && g.R % TK == 0 && op_ok(g.Y, g.yb, g.yj, g.yr, YR);
    const bool out_fast = g.J % 4 == 0 && (uintptr_t)g.out % 16 == 0;
    if (x_fast && y_fast && out_fast) { launch_mfma_impl<T, XR, YR, Cfg, true>(g); return; }
    // A reduction that is not whole k-tiles, or operands that are not aligned: the checked body loads element by element
    // (bf16 [1000,1000]x[1000,1000] ran at 23 TFLOP/s).  A product of some size copies such an operand first - a few
    // microseconds - with its reduction padded with zeros to whole k-tiles, which changes no bit of the result: the checked
    // body multiplies the same zeros, and the reduction is cut into chunks as it would be without the copy.
    const uint32_t Rp = (uint32_t)(cdiv(g.R, TK) * TK);
    const uint32_t pitch_x = (uint32_t)(cdiv(g.I, 8) * 8), pitch_y = (uint32_t)(cdiv(g.J, 8) * 8);
    const size_t per_x = x_fast ? 0 : (XR ? (size_t)g.I * Rp : (size_t)Rp * pitch_x);
    const size_t per_y = y_fast ? 0 : (YR ? (size_t)g.J * Rp : (size_t)Rp * pitch_y);
    const size_t bytes_x = (per_x * g.batch * sizeof(T) + 255) & ~(size_t)255, bytes_y = per_y * g.batch * sizeof(T);
    const bool repack = out_fast && !capture_open() && !prog_recording() && g.batch <= 65535 &&
                        (double)g.I * g.J * g.R * g.batch >= (double)(1 << 24) && per_x < (1ull << 31) && per_y < (1ull << 31) &&
                        bytes_x + bytes_y <= ((size_t)1 << 30);
    if (!repack) { launch_mfma_impl<T, XR, YR, Cfg, false>(g); return; }
    unsigned char* buf = (unsigned char*)scratch(bytes_x + bytes_y, 1);
    if (!buf) return;
    GemmArgs p = g;
    if (!x_fast) {
        hipLaunchKernelGGL((gemm_repack_kernel<T, XR>), dim3((unsigned)cdiv(per_x, 256), g.batch), dim3(256), 0, stream(), (const T*)g.X, (T*)buf,
                           g.I, g.R, Rp, pitch_x, g.xb, g.xi, g.xr);
        MXH_LAUNCH_CHECK("gemm_repack");
        p.X = buf; p.xb = (int64_t)per_x;
        if (XR) { p.xi = Rp; p.xr = 1; } else { p.xi = 1; p.xr = pitch_x; }
    }
    if (!y_fast) {
        hipLaunchKernelGGL((gemm_repack_kernel<T, YR>), dim3((unsigned)cdiv(per_y, 256), g.batch), dim3(256), 0, stream(), (const T*)g.Y,
                           (T*)(buf + bytes_x), g.J, g.R, Rp, pitch_y, g.yb, g.yj, g.yr);
        MXH_LAUNCH_CHECK("gemm_repack");
        p.Y = buf + bytes_x; p.yb = (int64_t)per_y;
        if (YR) { p.yj = Rp; p.yr = 1; } else { p.yj = 1; p.yr = pitch_y; }
    }
    p.R = Rp;
    launch_mfma_impl<T, XR, YR, Cfg, true>(p, nullptr, g.R);
}

// ---- small shapes (the per-thread and per-block dot kernels are in gemm_small.hpp) -------------------
// One wave per output element (gemm_wavedot_body in gemm_small.hpp).  For few outputs with a long reduction.
template <class T>
__global__ __launch_bounds__(GB) void gemm_wavedot_kernel(GemmArgs g) {
    gemm_wavedot_body<T>(g, (size_t)blockIdx.x * (GB / WAVE) + threadIdx.x / WAVE, threadIdx.x % WAVE, nullptr);
}

// byte range of a strided matmul operand: `rows` by `cols` elements at the given element strides
static Extent operand_extent(const void* base, size_t rows, int64_t row_stride, size_t cols, int64_t col_stride, size_t batch, int64_t batch_stride, size_t esz) {
    size_t span = (rows ? (rows - 1) * (size_t)row_stride : 0) + (cols ? (cols - 1) * (size_t)col_stride : 0) + (batch ? (batch - 1) * (size_t)batch_stride : 0);
    return Extent{(uintptr_t)base, (uintptr_t)base + (span + 1) * esz};
}
static bool positive_strides(const GemmArgs& g) { return g.xb >= 0 && g.xi >= 0 && g.xr >= 0 && g.yb >= 0 && g.yr >= 0 && g.yj >= 0; }

// While a capture is open: a one-thread-per-output f32 product offered to the open chain as a producer over the flat
// space of its outputs (true: do not launch).
static bool fuse_thread_dot(const GemmArgs& g, size_t outputs) {
    // (a chain takes reductions of at most 16 terms; a resident step program any this dispatch sends here)
    if (!capture_open() || g.batch != 1 || g.R > 256 || outputs >= (1u << 24) || !positive_strides(g)) return false;
    FuseCmd c;
    std::memset((void*)&c, 0, sizeof(c));
    c.out = g.out;
    c.in[0] = g.X;
    c.in[1] = g.Y;
    c.os[0] = 1;
    c.is[0][0] = g.xi; c.is[0][1] = g.xr;
    c.is[1][0] = g.yr; c.is[1][1] = g.yj;
    c.op = FUSE_OP_DOT;
    c.nin = 2;
    c.dims[0] = g.J; c.dims[1] = g.R;
    return fuse_record_dot(c, outputs, operand_extent(g.X, g.I, g.xi, g.R, g.xr, 1, 0, sizeof(float)),
                           operand_extent(g.Y, g.R, g.yr, g.J, g.yj, 1, 0, sizeof(float)), [g, outputs] {
                               hipLaunchKernelGGL(gemm_thread_kernel<float>, dim3(cdiv(outputs, GB)), dim3(GB), 0, stream(), g);
                               MXH_LAUNCH_CHECK("gemm_thread");
                           }, g.R <= 16);
}
// The same for a product of a handful of outputs with a long reduction: a stage of the chain's tail.
static bool fuse_block_dot(const GemmArgs& g, size_t outputs, bool rows) {
    if (!capture_open() || outputs > 8 || g.R > 65536 || !positive_strides(g)) return false;
    static_assert(sizeof(GemmArgs) <= FUSE_TAIL_ARG_BYTES, "a tail stage holds a matmul's arguments");
    const Extent in[2] = {operand_extent(g.X, g.I, g.xi, g.R, g.xr, g.batch, g.xb, sizeof(float)),
                          operand_extent(g.Y, g.R, g.yr, g.J, g.yj, g.batch, g.yb, sizeof(float))};
    const Extent out{(uintptr_t)g.out, (uintptr_t)g.out + outputs * sizeof(float)};
    return fuse_record_tail(TAIL_DOT, rows ? 1 : 0, &g, sizeof(g), in, 2, out, outputs);
}

// ... and for a handful of outputs that the dispatch gives a wave each (a reduction of a few hundred to a few thousand terms)
static bool fuse_wave_dot(const GemmArgs& g, size_t outputs) {
    if (!capture_open() || outputs > 16 || g.batch != 1 || !positive_strides(g)) return false;
    const Extent in[2] = {operand_extent(g.X, g.I, g.xi, g.R, g.xr, 1, 0, sizeof(float)), operand_extent(g.Y, g.R, g.yr, g.J, g.yj, 1, 0, sizeof(float))};
    const Extent out{(uintptr_t)g.out, (uintptr_t)g.out + outputs * sizeof(float)};
    return fuse_record_tail(TAIL_DOT, 2, &g, sizeof(g), in, 2, out, outputs);
}

__global__ __launch_bounds__(256) void gemm_rowsdot_kernel(GemmArgs g) {
    __shared__ float part[4 * 256 / WAVE];
    gemm_rowsdot_any<256>(g, threadIdx.x, part);
}

// A few output rows against a row-major Y ([1..8, R] x [R, J]: a batch of one to eight through a weight matrix).  The
// product is Y read once, so the kernel is a stream over Y's rows: a lane owns one 16-byte vector of columns, a wave 64
// of them (1 KB of every row) over its own run of r_chunk rows, eight rows in flight; X's elements are the same for the
// whole wave.  Every wave writes its f32 partial rows to part[chunk][I * J], and gemm_fold_kernel adds the chunks in order.
// (One wave per output, lanes striding down a column of Y, reads 4 bytes of every cache line it touches: [1,4096] x
// [4096,4096] in f32 took 100 us, 8 % of what the 64 MB of Y allow.)
template <class T, int MI>
__global__ __launch_bounds__(256) void gemm_fewrows_kernel(GemmArgs g) {
    constexpr int VEC = 16 / sizeof(T), U = 8;
    const uint32_t lane = threadIdx.x % WAVE;
    const uint32_t w = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const uint32_t j = (blockIdx.x * WAVE + lane) * VEC;
    const uint32_t chunk = blockIdx.y * (256 / WAVE) + w;
    if (chunk >= g.splits) return;
    const bool live = j < g.J;
    const uint32_t r0 = chunk * g.r_chunk, r1 = r0 + g.r_chunk < g.R ? r0 + g.r_chunk : g.R;
    float acc[MI][VEC];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[i][e] = 0.0f;
    const T* y = (const T*)g.Y + (live ? j : 0);
    const T* x = (const T*)g.X;
    auto rows = [&](uint32_t r, auto count) {
        constexpr int N = decltype(count)::value;
        AVec<T, VEC> v[N];
#pragma unroll
        for (int u = 0; u < N; ++u) v[u] = *(const AVec<T, VEC>*)(y + (int64_t)(r + u) * g.yr);
#pragma unroll
        for (int u = 0; u < N; ++u)
#pragma unroll
            for (int i = 0; i < MI; ++i) {
                const float a = (uint32_t)i < g.I ? Elem<T>::ld(x[(int64_t)i * g.xi + (int64_t)(r + u) * g.xr]) : 0.0f;
#pragma unroll
                for (int e = 0; e < VEC; ++e) acc[i][e] += a * Elem<T>::ld(v[u].v[e]);
            }
    };
    uint32_t r = r0;
    for (; r + U <= r1; r += U) rows(r, std::integral_constant<int, U>{});
    for (; r < r1; ++r) rows(r, std::integral_constant<int, 1>{});
    if (!live) return;
    float* dst = g.part + (size_t)chunk * g.I * g.J + j;
#pragma unroll
    for (int i = 0; i < MI; ++i)
        if ((uint32_t)i < g.I) {
            AVec<float, VEC> o;
#pragma unroll
            for (int e = 0; e < VEC; ++e) o.v[e] = acc[i][e];
            *(AVec<float, VEC>*)(dst + (size_t)i * g.J) = o;
        }
}

// false: the shape is not this kernel's
template <class T>
bool launch_fewrows(GemmArgs g) {
    constexpr int VEC = 16 / sizeof(T);
    // (f32, one or two rows: from three rows, and for the 16-bit dtypes from the first, the MFMA tiles with bounded
    // rows are faster - bf16 one row 21 us here, 14 us there)
    if (sizeof(T) != 4 || g.batch != 1 || g.I > 2 || g.yj != 1 || g.J < 256 || g.R < 256 || g.J % VEC != 0 || g.yr % VEC != 0 || g.yr < 0 ||
        (uintptr_t)g.Y % 16 != 0 || capture_open() || prog_recording())
        return false;
    const uint32_t colgroups = (uint32_t)cdiv((size_t)g.J / VEC, (size_t)WAVE);
    // about four waves per CU, at least 32 rows each
    uint32_t chunks = (uint32_t)std::min<size_t>(std::max<size_t>(cdiv((size_t)1024, (size_t)colgroups), 1), g.R / 32);
    g.r_chunk = (uint32_t)cdiv((size_t)g.R, (size_t)chunks);
    chunks = (uint32_t)cdiv((size_t)g.R, (size_t)g.r_chunk);
    g.splits = chunks;
    const size_t n_out = (size_t)g.I * g.J;
    g.part = (float*)scratch(chunks * n_out * sizeof(float) + 256);
    if (!g.part) return true;          // status is set
    const dim3 grid(colgroups, (unsigned)cdiv((size_t)chunks, (size_t)(256 / WAVE)));
    if (g.I == 1) hipLaunchKernelGGL((gemm_fewrows_kernel<T, 1>), grid, dim3(256), 0, stream(), g);
    else if (g.I == 2) hipLaunchKernelGGL((gemm_fewrows_kernel<T, 2>), grid, dim3(256), 0, stream(), g);
    else if (g.I <= 4) hipLaunchKernelGGL((gemm_fewrows_kernel<T, 4>), grid, dim3(256), 0, stream(), g);
    else hipLaunchKernelGGL((gemm_fewrows_kernel<T, 8>), grid, dim3(256), 0, stream(), g);
    MXH_LAUNCH_CHECK("gemm_fewrows");
    hipLaunchKernelGGL(gemm_fold_kernel<T>, dim3((unsigned)cdiv(n_out, (size_t)256)), dim3(256), 0, stream(), g.part, (T*)g.out, n_out, chunks);
    MXH_LAUNCH_CHECK("gemm_fold");
    return true;
}

// The same few rows against a matrix given transposed ([2..8, R] x W^T with W [J, R] row-major: a linear layer's
// forward): a wave per output column reads its row of W once, with the rows of X beside it (X is small and stays in
// cache), 16-byte vectors down the reduction, one sum per output row in a lane, a butterfly per row at the end.  The
// 64-row MFMA tiles took 52 us for [8,4096] x [4096,4096]^T: two latency-bound blocks per CU.
template <class T, int MI, int NJ>
__global__ __launch_bounds__(256) void gemm_fewrows_t_kernel(GemmArgs g) {
    // NJ output columns to a wave: a vector of X is loaded once for NJ rows of W
    constexpr int VEC = 16 / sizeof(T), U = MI * NJ <= 8 ? 4 : MI * NJ <= 16 ? 2 : 1;
    const uint32_t lane = threadIdx.x % WAVE;
    const uint32_t j0 = (blockIdx.x * (256 / WAVE) + __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE)) * NJ;
    if (j0 >= g.J) return;
    const T* x = (const T*)g.X;
    float acc[MI][NJ];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int c = 0; c < NJ; ++c) acc[i][c] = 0.0f;
    auto step = [&](uint32_t r) {
        AVec<T, VEC> yv[NJ];
#pragma unroll
        for (int c = 0; c < NJ; ++c) yv[c] = *(const AVec<T, VEC>*)((const T*)g.Y + (int64_t)(j0 + c < g.J ? j0 + c : j0) * g.yj + r);
#pragma unroll
        for (int i = 0; i < MI; ++i) {
            if ((uint32_t)i < g.I) {
                const AVec<T, VEC> xv = *(const AVec<T, VEC>*)(x + (int64_t)i * g.xi + r);
#pragma unroll
                for (int c = 0; c < NJ; ++c)
#pragma unroll
                    for (int e = 0; e < VEC; ++e) acc[i][c] += Elem<T>::ld(xv.v[e]) * Elem<T>::ld(yv[c].v[e]);
            }
        }
    };
    uint32_t r = lane * VEC;
    for (; r + (U - 1) * WAVE * VEC < g.R; r += U * WAVE * VEC) {
#pragma unroll
        for (int u = 0; u < U; ++u) step(r + u * WAVE * VEC);
    }
    for (; r < g.R; r += WAVE * VEC) step(r);
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int c = 0; c < NJ; ++c) {
            float t = acc[i][c];
#pragma unroll
            for (int off = 32; off > 0; off >>= 1) t += __shfl_xor(t, off, WAVE);
            if (lane == 0 && (uint32_t)i < g.I && j0 + c < g.J) ((T*)g.out)[(size_t)i * g.J + j0 + c] = Elem<T>::st(t);
        }
}

template <class T>
bool launch_fewrows_t(const GemmArgs& g) {
    constexpr int VEC = 16 / sizeof(T);
    // (two rows: from three the MFMA tiles with bounded rows are faster - f32 four rows 24 us here, 21 us there)
    if (g.batch != 1 || g.I != 2 || g.yr != 1 || g.xr != 1 || g.R < 512 || g.R % VEC != 0 || g.yj % VEC != 0 || g.xi % VEC != 0 ||
        g.yj < 0 || g.xi < 0 || (uintptr_t)g.Y % 16 != 0 || (uintptr_t)g.X % 16 != 0 || prog_recording())
        return false;
    // one column a wave: with two or four (X loaded once for several rows of W) the fewer waves cost more than the
    // loads saved - [8,4096] x [4096,4096]^T in f32 42 -> 58 us, bf16 26 -> 37 us
    auto grid = [&](int nj) { return dim3((unsigned)cdiv(cdiv((size_t)g.J, (size_t)nj), (size_t)(256 / WAVE))); };
    if (g.I == 2) hipLaunchKernelGGL((gemm_fewrows_t_kernel<T, 2, 1>), grid(1), dim3(256), 0, stream(), g);
    else if (g.I <= 4) hipLaunchKernelGGL((gemm_fewrows_t_kernel<T, 4, 1>), grid(1), dim3(256), 0, stream(), g);
    else hipLaunchKernelGGL((gemm_fewrows_t_kernel<T, 8, 1>), grid(1), dim3(256), 0, stream(), g);
    MXH_LAUNCH_CHECK("gemm_fewrows_t");
    return true;
}

template <class T>
void gemm_dispatch(GemmArgs g) {
    if (g.I == 0 || g.J == 0 || g.batch == 0) return;
    size_t outputs = (size_t)g.I * g.J * g.batch;
    // (16-bit dtypes: a reduction shorter than a k-tile would be a ragged tile for the MFMA kernel, i.e. its checked body)
    const bool short_r16 = sizeof(T) == 2 && g.R < 64 && !prog_recording() && gemm_thread_vec_ok<T>(g);
    if (g.R <= 16 || short_r16 || (g.I < 16 && g.J < 16 && g.R < 256)) {
        if constexpr (std::is_same<T, float>::value) {
            const bool small = cdiv(outputs, GB) <= PROG_MAX_GRID && (size_t)g.R * outputs <= PROG_MAX_ELEMS;
            if (prog_recording() && !small) prog_abandon();
            if (fuse_thread_dot(g, outputs)) return;
            if (prog_recording()) prog_record(prog_kid(PF_GEMM_THREAD, 0), (unsigned)cdiv(outputs, GB), &g, sizeof(g));
        }
        if (!prog_recording() && gemm_thread_vec_ok<T>(g)) {
            constexpr int VEC = 16 / sizeof(T);
            hipLaunchKernelGGL(gemm_thread_vec_kernel<T>, dim3((unsigned)cdiv((size_t)g.I * (g.J / VEC), (size_t)GB), g.batch), dim3(GB), 0, stream(), g);
            MXH_LAUNCH_CHECK("gemm_thread_vec");
            return;
        }
        hipLaunchKernelGGL(gemm_thread_kernel<T>, dim3(cdiv(outputs, GB)), dim3(GB), 0, stream(), g);
        MXH_LAUNCH_CHECK("gemm_thread");
        return;
    }
    // (up to eight outputs from 1024 terms on: such a product is a stage of a captured chain's tail, where one wave per
    // output would leave most of the work-group idle)
    if (outputs <= 64 && (g.R >= 4096 || (outputs <= 8 && g.R >= 1024))) {
        const bool wide = blockdot_threads(g.R) == 1024;
        if constexpr (std::is_same<T, float>::value) {
            const bool small = (size_t)g.R * outputs <= PROG_MAX_ELEMS;
            if (prog_recording() && !small) prog_abandon();
            const bool rows = rowsdot_applies(g);        // [1,R] x [R,J]: one block, vector loads
            if (!wide && fuse_block_dot(g, outputs, rows)) return;
            if (rows) {
                if (prog_recording()) prog_record(prog_kid(PF_GEMM_ROWSDOT, 0), 1, &g, sizeof(g));
                hipLaunchKernelGGL(gemm_rowsdot_kernel, dim3(1), dim3(256), 0, stream(), g);
                MXH_LAUNCH_CHECK("gemm_rowsdot");
                return;
            }
            if (prog_recording()) prog_record(prog_kid(PF_GEMM_BLOCKDOT, 0), (unsigned)outputs, &g, sizeof(g));
        }
        if (wide) hipLaunchKernelGGL((gemm_blockdot_kernel<T, 1024>), dim3((unsigned)outputs), dim3(1024), 0, stream(), g);
        else hipLaunchKernelGGL((gemm_blockdot_kernel<T, 256>), dim3((unsigned)outputs), dim3(256), 0, stream(), g);
        MXH_LAUNCH_CHECK("gemm_blockdot");
        return;
    }
    if (launch_fewrows<T>(g) || launch_fewrows_t<T>(g)) return;
    // (a few rows against a large row-major Y are not for the kernel below, whose lanes would stride down Y's columns)
    // (nor is a long reduction along which both operands are strided, a weight gradient [128,10000]^T x [10000,10]: every
    // lane of a wave would read a cache line of its own, 74 us; the tiles below cut the reduction over the chip)
    const bool both_strided = g.xr != 1 && g.yr != 1 && g.R >= 2048 && g.I >= 32;
    if (outputs <= 4096 && (g.I < 32 || g.J < 32) && !(g.yj == 1 && g.J >= 256 && g.R >= 256) && !both_strided) {
        if constexpr (std::is_same<T, float>::value) {
            if (prog_recording()) prog_abandon();
            if (fuse_wave_dot(g, outputs)) return;
        }
        hipLaunchKernelGGL(gemm_wavedot_kernel<T>, dim3(cdiv(outputs, GB / WAVE)), dim3(GB), 0, stream(), g);
        MXH_LAUNCH_CHECK("gemm_wavedot");
        return;
    }
    bool xr = g.xr == 1, yr = g.yr == 1;
    bool xi = g.xi == 1, yj = g.yj == 1;
    // 256x256 tiles when they fill the chip about as well as 128x128 ones would
    size_t big_blocks = (size_t)cdiv(g.I, 256) * cdiv(g.J, 256) * g.batch;
    // Few output columns, or a reduction of a few k-tiles (prologue and epilogue are then most of a block's life, and
    // many small blocks overlap them): the 64-column tiles.  Measured on the convolution layer's f32 products
    // [100352,576]x[576,64], [100352,64]x[64,576], [576,100352]x[100352,64]: 76 / 112 / 106 us with 64x64 tiles
    // (four blocks per CU), 86 / 116 / 144 us with 128x64, 196 / 124 / 196 us with 128x128, 340 / 137 / 339 us with
    // 256x256.
    constexpr uint32_t TKE = TK_BYTES / sizeof(T);
    // At most 64 output rows (a small batch through a weight matrix): a 128-row tile would compute mostly rows that do
    // not exist - [16,4096] x [4096,4096] in f32 took 49 us, the time of 128 rows.
    bool tall = (g.I >= 128 && (g.J <= 64 || g.R <= 4 * TKE)) || g.I <= 64;
    bool big = !tall && g.I >= 256 && g.J >= 256 && big_blocks >= 192;
    const bool flat = g.I <= 32 && g.J >= 128;
#define MXH_GEMM_CASE(XR, YR) (big ? launch_mfma<T, XR, YR, typename Cfgs<T>::Big>(g) : flat ? launch_mfma<T, XR, YR, typename Cfgs<T>::Flat>(g) : tall ? launch_mfma<T, XR, YR, typename Cfgs<T>::Tall>(g) : launch_mfma<T, XR, YR, typename Cfgs<T>::Small>(g))
    if (xr && yr) MXH_GEMM_CASE(true, true);
    else if (xr && yj) MXH_GEMM_CASE(true, false);
    else if (xi && yr) MXH_GEMM_CASE(false, true);
    else if (xi && yj) MXH_GEMM_CASE(false, false);
    else {
        // no unit stride on one operand: correct but slow
        if constexpr (std::is_same<T, float>::value)
            if (prog_recording() && cdiv(outputs, GB) <= PROG_MAX_GRID && (size_t)g.R * outputs <= PROG_MAX_ELEMS)
                prog_record(prog_kid(PF_GEMM_THREAD, 0), (unsigned)cdiv(outputs, GB), &g, sizeof(g));
        hipLaunchKernelGGL(gemm_thread_kernel<T>, dim3(cdiv(outputs, GB)), dim3(GB), 0, stream(), g);
        MXH_LAUNCH_CHECK("gemm_thread");
    }
#undef MXH_GEMM_CASE
}

// The Conv2d layer's two products with the column matrix, the matrix gathered from the input instead of stored.
//   transposed == 0: out[M, n] = cols x rhs,    rhs [K, n]      (forward: nn/layers/conv.rs:222)
//   transposed != 0: out[K, n] = cols^T x rhs,  rhs [M, n]      (weight gradient: conv.rs:279)
// with M = B*oh*ow, K = C*kh*kw; md as conv2d_im2col reads it; rs: element strides of rhs (one of them 1).
static void cols_matmul(const size_t* md, int transposed, const float* in, const float* rhs, size_t n, const size_t* rs, float* out) {
    if (!md || !rs) { set_status(ERR_INVALID, "conv2d_cols_matmul: null metadata"); return; }
    const size_t B = md[0], C = md[1], H = md[2], W = md[3], kh = md[4], kw = md[5], oh = md[6], ow = md[7];
    const size_t ph = md[8], pw = md[9], sh = md[10], sw = md[11];
    const size_t M = B * oh * ow, K = C * kh * kw;
    if (M == 0 || K == 0 || n == 0) return;
    if (!in || !rhs || !out) { set_status(ERR_INVALID, "conv2d_cols_matmul: null buffer"); return; }
    if (H == 0 || W == 0) { set_status(ERR_INVALID, "conv2d_cols_matmul: empty input plane"); return; }
    const size_t lim = (size_t)1 << 31;
    if (M * K >= lim || B * C * H * W >= lim || n >= lim || ph >= lim || pw >= lim || sh * oh >= lim || sw * ow >= lim) {
        set_status(ERR_TOO_LARGE, "conv2d_cols_matmul: 2^31 or more entries");
        return;
    }
    if (rs[0] != 1 && rs[1] != 1) { set_status(ERR_UNSUPPORTED, "conv2d_cols_matmul: rhs needs a unit stride"); return; }
    if (prog_recording()) prog_abandon();
    ColsView v;
    v.in = in;
    v.K = (uint32_t)K; v.P = (uint32_t)(oh * ow);
    v.H = (uint32_t)H; v.W = (uint32_t)W; v.HW = (uint32_t)(H * W); v.CHW = (uint32_t)(C * H * W);
    v.sh = (uint32_t)sh; v.sw = (uint32_t)sw; v.ph = (int32_t)ph; v.pw = (int32_t)pw;
    v.d_P = make_fastdiv(v.P); v.d_khkw = make_fastdiv((uint32_t)(kh * kw));
    v.d_kw = make_fastdiv((uint32_t)kw); v.d_ow = make_fastdiv((uint32_t)ow);
    const bool vec4 = K % 4 == 0 && ow % 4 == 0;            // (then P % 4 == 0 as well)
    GemmArgs g;
    std::memset((void*)&g, 0, sizeof(g));
    g.X = in;                      // not addressed through the strides below: the tiles are gathered
    g.Y = rhs;
    g.out = out;
    g.batch = 1;
    g.J = (uint32_t)n;
    g.yr = (int64_t)rs[0]; g.yj = (int64_t)rs[1];
    if (!transposed) { g.I = (uint32_t)M; g.R = (uint32_t)K; g.xi = (int64_t)K; g.xr = 1; }
    else { g.I = (uint32_t)K; g.R = (uint32_t)M; g.xi = 1; g.xr = (int64_t)K; }
    // the choices gemm_dispatch makes for a stored matrix of this shape, so that both ways are the same arithmetic
    constexpr uint32_t TK = TK_BYTES / sizeof(float);
    const bool tall = (g.I >= 128 && (g.J <= 64 || g.R <= 4 * TK)) || g.I <= 64;
    const bool yr = g.yr == 1;
    auto fast_of = [&](int rows_y) {
        const bool span = g.yj >= 0 && g.yr >= 0 && ((int64_t)rows_y * g.yj + (int64_t)TK * g.yr) * 4 < (1ll << 31);
        const bool y_ok = yr ? ((uintptr_t)g.Y % 16 == 0 && g.yj % 4 == 0) : true;
        return span && y_ok && g.R % TK == 0 && g.J % 4 == 0 && (uintptr_t)g.out % 16 == 0;
    };
    // (one by one only with the checked body: odd widths are not the shapes to tune for)
#define MXH_COLS_CASE(XR, YR, CFG)                                                                  \
    (!vec4 ? launch_mfma_impl<float, XR, YR, CFG, false, 1>(g, &v)                                  \
           : fast_of(CFG::TN) ? launch_mfma_impl<float, XR, YR, CFG, true, 2>(g, &v) : launch_mfma_impl<float, XR, YR, CFG, false, 2>(g, &v))
    using TallCfg = Cfgs<float>::Tall;
    using SmallCfg = Cfgs<float>::Small;
#define MXH_COLS_CFG(XR, YR) (tall ? MXH_COLS_CASE(XR, YR, TallCfg) : MXH_COLS_CASE(XR, YR, SmallCfg))
    if (!transposed) { if (yr) MXH_COLS_CFG(true, true); else MXH_COLS_CFG(true, false); }
    else { if (yr) MXH_COLS_CFG(false, true); else MXH_COLS_CFG(false, false); }
#undef MXH_COLS_CFG
#undef MXH_COLS_CASE
}

}  // namespace mxh

using namespace mxh;

extern "C" void hip_conv2d_cols_matmul_f32(const size_t* metadata, int transposed, const float* input, const float* rhs, size_t n,
                                           const size_t* rhs_strides, float* out) { MXH_API;
    cols_matmul(metadata, transposed, input, rhs, n, rhs_strides, out);
}

// out[b][j][p] = (X[b*P + p][:] . W[j][:]) + bias[j] for X [M, K] and W [J, K], both row-major: 1 when it ran, 0 when the
// shapes are not for it (nothing queued)
extern "C" int hip_conv2d_forward_product_f32(size_t M, size_t K, size_t J, size_t P, const float* x, const float* w, const float* bias,
                                              float* out) {
    MXH_API_INT;
    using Cfg = Cfgs<float>::Tall;
    constexpr size_t TK = TK_BYTES / sizeof(float);
    if (!x || !w || !bias || !out || M == 0 || K == 0 || J == 0 || P == 0) return 0;
    if (M % P != 0 || M % Cfg::TM != 0 || J % Cfg::TN != 0 || K % TK != 0 || M >= (1ull << 31) || K >= (1ull << 31) || J > 64) return 0;
    if ((uintptr_t)x % 16 || (uintptr_t)w % 16 || (uintptr_t)bias % 16 || M * J >= (1ull << 31) || M * K >= (1ull << 62)) return 0;
    if (((int64_t)Cfg::TM * (int64_t)K + (int64_t)TK) * 4 >= (1ll << 31)) return 0;      // per-thread offsets inside a tile are 32-bit
    if (prog_recording()) prog_abandon();
    GemmArgs g;
    std::memset((void*)&g, 0, sizeof(g));
    g.X = x; g.Y = w; g.out = out;
    g.xb = 0; g.xi = (int64_t)K; g.xr = 1;
    g.yb = 0; g.yr = 1; g.yj = (int64_t)K;
    g.I = (uint32_t)M; g.J = (uint32_t)J; g.R = (uint32_t)K; g.batch = 1;
    g.tiles_i = (uint32_t)(M / Cfg::TM);
    g.tiles_j = (uint32_t)(J / Cfg::TN);
    g.splits = 1;
    g.r_chunk = g.R;
    g.part = nullptr;
    if ((size_t)g.tiles_i * g.tiles_j <= 128) return 0;        // (few tiles: the plain product cuts the reduction over the chip)
    GemmEpi e;
    e.bias = bias;
    e.P = (uint32_t)P;
    e.d_P = make_fastdiv((uint32_t)P);
    using SX = Stager<float, true, Cfg::TM, Cfg::NT, false>;
    constexpr size_t lds_bytes = (size_t)2 * (Cfg::TM + Cfg::TN) * SX::PITCH * sizeof(float);
    static_assert(lds_bytes <= (64u << 10), "no attribute needed");
    hipLaunchKernelGGL(gemm_mfma_planes_kernel<Cfg>, dim3(g.tiles_i * g.tiles_j), dim3(Cfg::NT), lds_bytes, stream(), g, e);
    MXH_LAUNCH_CHECK("gemm_mfma_planes");
    return 1;
}

#define MXH_MATMUL_FOR(T, SUF)                                                                              \
    extern "C" void hip_matmul_##SUF(size_t num_els, const size_t* md, const T* a, const T* b, T* c) { MXH_API; \
        matmul_fwd<T>(num_els, md, a, b, c, [](GemmArgs g) { gemm_dispatch<T>(g); });                       \
    }                                                                                                       \
    extern "C" void hip_matmul_backward_##SUF(size_t na, size_t nb, const size_t* md, const T* go,          \
                                              const T* a, const T* b, T* ga, T* gb) { MXH_API;              \
        matmul_bwd<T>(na, nb, md, go, a, b, ga, gb, [](GemmArgs g) { gemm_dispatch<T>(g); });               \
    }

MXH_MATMUL_FOR(float, f32)
MXH_MATMUL_FOR(bf16_t, bf16)
MXH_MATMUL_FOR(f16_t, f16)
