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
// Large products run on MFMA (v_mfma_f32_32x32x16_bf16 / v_mfma_f32_32x32x2_f32): 128x128 output
// tile per 256-thread block, 2x2 waves, each wave a 64x64 patch = 2x2 MFMA tiles, f32 accumulate,
// one rounding at the end for bf16.  Operands sit in LDS as [row][k] with the reduction index
// contiguous, so a lane fetches its whole fragment with one 128-bit ds_read.
// Small or skinny products (the MLP's [10000,3]x[3,1] and its [3,10000]x[10000,1] gradient) use
// a thread-per-output kernel (bit-exact with the reference: k ascending, unfused f32) or a
// wave-per-output dot kernel.
#include "mxh.hpp"

namespace mxh {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

struct GemmArgs {
    const void* X;
    const void* Y;
    void* out;
    int64_t xb, xi, xr;   // element strides of X: batch, output row, reduction
    int64_t yb, yr, yj;   // element strides of Y: batch, reduction, output column
    uint32_t I, J, R, batch;
    uint32_t tiles_i, tiles_j;
};

template <class T> struct Elem;
template <> struct Elem<float> {
    static constexpr int VEC = 4;      // elements per 16-byte LDS fragment read
    static __device__ float ld(float v) { return v; }
    static __device__ float st(float v) { return v; }
    static __device__ float zero() { return 0.0f; }
};
template <> struct Elem<bf16_t> {
    static constexpr int VEC = 8;
    static __device__ float ld(bf16_t v) { return bf2f(v); }
    static __device__ bf16_t st(float v) { return f2bf(v); }
    static __device__ bf16_t zero() { return bf16_t{0}; }
};

constexpr int GB = 256;          // threads per block
constexpr int TM = 128, TN = 128;
constexpr int TK_BYTES = 128;    // reduction extent of one staged tile, in bytes per row

template <class T, int N> struct alignas(sizeof(T) * N) GVec { T v[N]; };

// ---- staging one 128 x TK operand tile into LDS as [row][TK + PAD] ---------------------------------
// `rows` is the operand's output index (i for X, j for Y).  RCONT: the reduction index has
// stride 1 in memory (natural); otherwise the row index has stride 1 and the tile is turned here.
template <class T, bool RCONT>
struct Stager {
    static constexpr int VEC = Elem<T>::VEC;
    static constexpr int TK = TK_BYTES / sizeof(T);
    static constexpr int PITCH = TK + VEC;                 // keeps 16-byte alignment, skews banks
    static constexpr int NV = TM * TK / VEC / GB;          // 16-byte units per thread (4)
    GVec<T, VEC> reg[NV];

    // natural: unit u → (row, kv);  turned: unit u → (r-group of VEC, row)
    __device__ void load(const T* __restrict__ base, int64_t s_row, int64_t s_red, uint32_t row0, uint32_t red0,
                         uint32_t nrows, uint32_t nred, bool fast) {
        const int t = threadIdx.x;
        if constexpr (RCONT) {
            constexpr int KV = TK / VEC;   // vectors per row
#pragma unroll
            for (int u = 0; u < NV; ++u) {
                int id = t + u * GB;
                uint32_t row = row0 + id / KV, red = red0 + (id % KV) * VEC;
                const T* p = base + (int64_t)row * s_row + red;
                if (fast) {
                    reg[u] = *(const GVec<T, VEC>*)p;
                } else {
#pragma unroll
                    for (int e = 0; e < VEC; ++e)
                        reg[u].v[e] = (row < nrows && red + e < nred) ? p[e] : Elem<T>::zero();
                }
            }
        } else {
            // lanes run along the row index (stride 1 in memory); each unit gathers VEC reduction
            // steps of one row so that the LDS write is again one 16-byte [row][k..k+VEC) vector.
            constexpr int RG = TK / VEC;   // reduction groups per tile
#pragma unroll
            for (int u = 0; u < NV; ++u) {
                int id = t + u * GB;
                uint32_t row = row0 + id % TM, red = red0 + (id / TM) * VEC;
                const T* p = base + (int64_t)row + (int64_t)red * s_red;
                (void)RG;
#pragma unroll
                for (int e = 0; e < VEC; ++e)
                    reg[u].v[e] = (fast || (row < nrows && red + e < nred)) ? p[(int64_t)e * s_red] : Elem<T>::zero();
            }
        }
    }
    __device__ void store(T* lds) const {
        const int t = threadIdx.x;
#pragma unroll
        for (int u = 0; u < NV; ++u) {
            int id = t + u * GB;
            int row, kk;
            if constexpr (RCONT) { constexpr int KV = TK / VEC; row = id / KV; kk = (id % KV) * VEC; }
            else { row = id % TM; kk = (id / TM) * VEC; }
            *(GVec<T, VEC>*)(lds + row * PITCH + kk) = reg[u];
        }
    }
};

template <class T> struct Mma;
template <> struct Mma<bf16_t> {
    static __device__ void run(const GVec<bf16_t, 8>& a, const GVec<bf16_t, 8>& b, f32x16& c) {
        c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    }
};
template <> struct Mma<float> {
    // one 16-byte fragment feeds four 32x32x2 steps; lane (row, h) holds k = 4h .. 4h+3 of an
    // 8-wide slice, and step e pairs element e of both operands — any fixed pairing of k is valid.
    static __device__ void run(const GVec<float, 4>& a, const GVec<float, 4>& b, f32x16& c) {
#pragma unroll
        for (int e = 0; e < 4; ++e) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a.v[e], b.v[e], c, 0, 0, 0);
    }
};

template <class T, bool XR, bool YR>
__global__ __launch_bounds__(GB) void gemm_mfma_kernel(GemmArgs g) {
    using SX = Stager<T, XR>;
    using SY = Stager<T, YR>;
    constexpr int VEC = Elem<T>::VEC;
    constexpr int TK = SX::TK;
    constexpr int PITCH = SX::PITCH;
    __shared__ __attribute__((aligned(16))) T lds_x[TM * PITCH];
    __shared__ __attribute__((aligned(16))) T lds_y[TN * PITCH];

    // block → (batch, tile_i, tile_j); neighbouring blocks share the X panel (tile_j fastest)
    uint32_t bid = blockIdx.x;
    uint32_t tj = bid % g.tiles_j;
    uint32_t rest = bid / g.tiles_j;
    uint32_t ti = rest % g.tiles_i;
    uint32_t b = rest / g.tiles_i;
    const uint32_t i0 = ti * TM, j0 = tj * TN;
    const T* X = (const T*)g.X + (int64_t)b * g.xb;
    const T* Y = (const T*)g.Y + (int64_t)b * g.yb;

    const int lane = threadIdx.x % WAVE, wave = threadIdx.x / WAVE;
    const int wm = wave / 2, wn = wave % 2;
    const int lrow = lane % 32, lk = (lane / 32) * VEC;

    f32x16 acc[2][2];
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[a][c][e] = 0.0f;

    // fast path: tile fully inside and every 16-byte access aligned
    auto vec_ok = [&](const T* p, int64_t s_row, bool rcont) {
        if (!rcont) return true;   // turned loads are scalar
        return ((uintptr_t)p % 16 == 0) && (s_row % VEC == 0);
    };
    const bool x_full = i0 + TM <= g.I, y_full = j0 + TN <= g.J;
    const bool x_al = vec_ok(X, g.xi, XR), y_al = vec_ok(Y, g.yj, YR);

    SX sx;
    SY sy;
    const uint32_t nk = (g.R + TK - 1) / TK;
    {
        bool kfull = TK <= g.R;
        sx.load(X, g.xi, g.xr, i0, 0, g.I, g.R, x_full && kfull && x_al);
        sy.load(Y, g.yj, g.yr, j0, 0, g.J, g.R, y_full && kfull && y_al);
    }
    for (uint32_t kt = 0; kt < nk; ++kt) {
        sx.store(lds_x);
        sy.store(lds_y);
        __syncthreads();
        if (kt + 1 < nk) {
            uint32_t r0 = (kt + 1) * TK;
            bool kfull = r0 + TK <= g.R;
            sx.load(X, g.xi, g.xr, i0, r0, g.I, g.R, x_full && kfull && x_al);
            sy.load(Y, g.yj, g.yr, j0, r0, g.J, g.R, y_full && kfull && y_al);
        }
#pragma unroll
        for (int s = 0; s < TK / (2 * VEC); ++s) {
            GVec<T, VEC> fa[2], fb[2];
#pragma unroll
            for (int a = 0; a < 2; ++a)
                fa[a] = *(const GVec<T, VEC>*)(lds_x + (wm * 64 + a * 32 + lrow) * PITCH + s * 2 * VEC + lk);
#pragma unroll
            for (int c = 0; c < 2; ++c)
                fb[c] = *(const GVec<T, VEC>*)(lds_y + (wn * 64 + c * 32 + lrow) * PITCH + s * 2 * VEC + lk);
#pragma unroll
            for (int a = 0; a < 2; ++a)
#pragma unroll
                for (int c = 0; c < 2; ++c) Mma<T>::run(fa[a], fb[c], acc[a][c]);
        }
        __syncthreads();
    }

    // accumulator element e of a 32x32 tile: row 8*(e/4) + 4*(lane/32) + e%4, column lane%32
    T* out = (T*)g.out + (int64_t)b * g.I * g.J;
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            uint32_t col = j0 + wn * 64 + c * 32 + lrow;
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                uint32_t row = i0 + wm * 64 + a * 32 + 8 * (e / 4) + 4 * (lane / 32) + (e % 4);
                if (row < g.I && col < g.J) out[(int64_t)row * g.J + col] = Elem<T>::st(acc[a][c][e]);
            }
        }
}

// ---- small shapes -----------------------------------------------------------------------------------
// One thread per output element, r ascending, multiply and add unfused: the reference's own
// order, so f32 results are bit-identical to it.
template <class T>
__global__ __launch_bounds__(GB) void gemm_thread_kernel(GemmArgs g) {
    size_t idx = (size_t)blockIdx.x * GB + threadIdx.x;
    size_t per = (size_t)g.I * g.J;
    if (idx >= per * g.batch) return;
    uint32_t b = (uint32_t)(idx / per);
    uint32_t rem = (uint32_t)(idx % per);
    uint32_t i = rem / g.J, j = rem % g.J;
    const T* x = (const T*)g.X + (int64_t)b * g.xb + (int64_t)i * g.xi;
    const T* y = (const T*)g.Y + (int64_t)b * g.yb + (int64_t)j * g.yj;
    float acc = 0.0f;
    for (uint32_t r = 0; r < g.R; ++r) acc = acc + Elem<T>::ld(x[(int64_t)r * g.xr]) * Elem<T>::ld(y[(int64_t)r * g.yr]);
    ((T*)g.out)[idx] = Elem<T>::st(acc);
}

// One wave per output element: lanes stride over r, 4 independent partial sums per lane, then a
// fixed shuffle tree.  For few outputs with a long reduction.
template <class T>
__global__ __launch_bounds__(GB) void gemm_wavedot_kernel(GemmArgs g) {
    size_t idx = (size_t)blockIdx.x * (GB / WAVE) + threadIdx.x / WAVE;
    size_t per = (size_t)g.I * g.J;
    const int lane = threadIdx.x % WAVE;
    float acc = 0.0f;
    bool live = idx < per * g.batch;
    if (live) {
        uint32_t b = (uint32_t)(idx / per);
        uint32_t rem = (uint32_t)(idx % per);
        uint32_t i = rem / g.J, j = rem % g.J;
        const T* x = (const T*)g.X + (int64_t)b * g.xb + (int64_t)i * g.xi;
        const T* y = (const T*)g.Y + (int64_t)b * g.yb + (int64_t)j * g.yj;
        float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
        uint32_t r = lane;
        for (; r + 3 * WAVE < g.R; r += 4 * WAVE) {
            a0 += Elem<T>::ld(x[(int64_t)r * g.xr]) * Elem<T>::ld(y[(int64_t)r * g.yr]);
            a1 += Elem<T>::ld(x[(int64_t)(r + WAVE) * g.xr]) * Elem<T>::ld(y[(int64_t)(r + WAVE) * g.yr]);
            a2 += Elem<T>::ld(x[(int64_t)(r + 2 * WAVE) * g.xr]) * Elem<T>::ld(y[(int64_t)(r + 2 * WAVE) * g.yr]);
            a3 += Elem<T>::ld(x[(int64_t)(r + 3 * WAVE) * g.xr]) * Elem<T>::ld(y[(int64_t)(r + 3 * WAVE) * g.yr]);
        }
        for (; r < g.R; r += WAVE) a0 += Elem<T>::ld(x[(int64_t)r * g.xr]) * Elem<T>::ld(y[(int64_t)r * g.yr]);
        acc = (a0 + a1) + (a2 + a3);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, WAVE);
    if (live && lane == 0) ((T*)g.out)[idx] = Elem<T>::st(acc);
}

template <class T>
void gemm_dispatch(GemmArgs g) {
    if (g.I == 0 || g.J == 0 || g.batch == 0) return;
    size_t outputs = (size_t)g.I * g.J * g.batch;
    if (g.R <= 16 || (g.I < 16 && g.J < 16 && g.R < 256)) {
        hipLaunchKernelGGL(gemm_thread_kernel<T>, dim3(cdiv(outputs, GB)), dim3(GB), 0, stream(), g);
        MXH_LAUNCH_CHECK("gemm_thread");
        return;
    }
    if (outputs <= 4096 && (g.I < 32 || g.J < 32)) {
        hipLaunchKernelGGL(gemm_wavedot_kernel<T>, dim3(cdiv(outputs, GB / WAVE)), dim3(GB), 0, stream(), g);
        MXH_LAUNCH_CHECK("gemm_wavedot");
        return;
    }
    g.tiles_i = cdiv(g.I, TM);
    g.tiles_j = cdiv(g.J, TN);
    size_t blocks = (size_t)g.tiles_i * g.tiles_j * g.batch;
    if (blocks >= (1ull << 31)) { set_status(ERR_TOO_LARGE, "matmul: too many tiles"); return; }
    bool xr = g.xr == 1, yr = g.yr == 1;
    bool xi = g.xi == 1, yj = g.yj == 1;
    dim3 grid((unsigned)blocks), blk(GB);
    if (xr && yr) hipLaunchKernelGGL((gemm_mfma_kernel<T, true, true>), grid, blk, 0, stream(), g);
    else if (xr && yj) hipLaunchKernelGGL((gemm_mfma_kernel<T, true, false>), grid, blk, 0, stream(), g);
    else if (xi && yr) hipLaunchKernelGGL((gemm_mfma_kernel<T, false, true>), grid, blk, 0, stream(), g);
    else if (xi && yj) hipLaunchKernelGGL((gemm_mfma_kernel<T, false, false>), grid, blk, 0, stream(), g);
    else {
        // no unit stride on one operand: correct but slow
        hipLaunchKernelGGL(gemm_thread_kernel<T>, dim3(cdiv(outputs, GB)), dim3(GB), 0, stream(), g);
    }
    MXH_LAUNCH_CHECK("gemm_mfma");
}

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
template <class T>
void matmul_fwd(size_t num_els, const size_t* md, const T* a, const T* b, T* c) {
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
    gemm_dispatch<T>(g);
}

// matmul.rs:124-268 — contiguous indexing, strides ignored, either gradient may be null.
template <class T>
void matmul_bwd(size_t num_els_a, size_t num_els_b, const size_t* md, const T* go, const T* a, const T* b, T* ga, T* gb) {
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
        gemm_dispatch<T>(g);
    }
    if (gb) {
        if (num_els_b % (k * n) != 0) { set_status(ERR_INVALID, "matmul_backward: num_els_b is not batch*k*n"); return; }
        GemmArgs g{};
        g.X = a + p.a_off; g.Y = go; g.out = gb;
        g.I = (uint32_t)k; g.J = (uint32_t)n; g.R = (uint32_t)m; g.batch = (uint32_t)(num_els_b / (k * n));
        g.xb = (int64_t)(m * k); g.xi = 1; g.xr = (int64_t)k;
        g.yb = (int64_t)(m * n); g.yr = (int64_t)n; g.yj = 1;
        gemm_dispatch<T>(g);
    }
}

}  // namespace mxh

using namespace mxh;

#define MXH_MATMUL_FOR(T, SUF)                                                                              \
    extern "C" void hip_matmul_##SUF(size_t num_els, const size_t* md, const T* a, const T* b, T* c) {      \
        matmul_fwd<T>(num_els, md, a, b, c);                                                                \
    }                                                                                                       \
    extern "C" void hip_matmul_backward_##SUF(size_t na, size_t nb, const size_t* md, const T* go,          \
                                              const T* a, const T* b, T* ga, T* gb) {                       \
        matmul_bwd<T>(na, nb, md, go, a, b, ga, gb);                                                        \
    }

MXH_MATMUL_FOR(float, f32)
MXH_MATMUL_FOR(bf16_t, bf16)
