// Softmax along one dim.  Replaces cuda_softmax_<T> of crates/maidenx_cuda/src/nn/activation/softmax.rs
// with the CPU semantics of crates/maidenx_cpu/src/nn/activation/softmax.rs:62-207.
// Metadata: dims[n] | strides[n] | offset; `dim` out of range means the last dim (:74).
// Per slice: m = max from -inf with `x > m` (NaNs never win), s = exp(-inf - m) + sum exp(x - m),
// out = exp(x - m) / s, written contiguously.  The maximum is exact; the sum is taken in f32 in a fixed
// tree order (the reference adds sequentially in the storage dtype), so results carry the tolerance of
// a reduction.  bf16 rounds x - m, exp and the final quotient like the reference does and keeps only the
// sum in f32.
//   contiguous, dim last : a wave (rows up to 2048) or a block per row; 16-byte loads, the row is held in
//                          registers between the three phases when it fits.
//   contiguous, dim inner: lanes run along the trailing dims (coalesced); short columns are walked by one
//                          thread each, long ones are split among the 16 waves of a block.
//   strided input        : one thread per slice with the reference's index rule (:120-136, the leading
//                          dims are decomposed from dim 0 upwards).
#include <algorithm>
#include <type_traits>

#include "elementwise.hpp"
#include "ops.hpp"
#include "mathfn.hpp"
#include "mxh.hpp"

namespace mxh {

template <class T> struct SM;
template <> struct SM<float> {
    static __device__ float ld(float v) { return v; }
    static __device__ float shifted(float x, float m) { return m_exp(x - m); }     // exp(x - m)
    static __device__ float fin(float e, float s) { return e / s; }
    static __device__ void keep(float& slot, float e) { slot = e; }
};
template <> struct SM<bf16_t> {
    static __device__ float ld(bf16_t v) { return bf2f(v); }
    static __device__ float shifted(float x, float m) { return bf2f(f2bf(m_exp(bf2f(f2bf(x - m))))); }
    static __device__ bf16_t fin(float e, float s) { return f2bf(e / bf2f(f2bf(s))); }
    static __device__ void keep(bf16_t& slot, float e) { slot = f2bf(e); }         // e is a bf16 value: exact
};

template <> struct SM<f16_t> {
    static __device__ float ld(f16_t v) { return h2f(v); }
    static __device__ float shifted(float x, float m) { return h2f(f2h(m_exp(h2f(f2h(x - m))))); }
    static __device__ f16_t fin(float e, float s) { return f2h(e / h2f(f2h(s))); }
    static __device__ void keep(f16_t& slot, float e) { slot = f2h(e); }
};

constexpr int SB = 256;

// Butterflies over groups of W consecutive lanes (W = 64: the wave).  A narrower group's sum is, bit for bit, what the
// wave-wide one gives when the other lanes hold 0: those steps add 0 to a sum of non-negative terms.
template <int W = WAVE>
__device__ inline float wave_max(float v) {
#pragma unroll
    for (int off = W / 2; off > 0; off >>= 1) {
        float o = __shfl_xor(v, off, WAVE);
        v = o > v ? o : v;
    }
    return v;
}
template <int W = WAVE>
__device__ inline float wave_sum(float v) {
#pragma unroll
    for (int off = W / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, WAVE);
    return v;
}

// rows of length D, TPR threads per row (8, 16, 32, WAVE or SB).  FITS: the row is held in registers, NREG vectors a
// thread (the host has checked D <= TPR * VEC * NREG), and exp(x - m) - a value of T - replaces x there, computed once;
// otherwise the row is read again from cache in each phase.
template <class T, int TPR, int VEC, int NREG, bool FITS>
__global__ __launch_bounds__(SB) void softmax_row_kernel(const T* __restrict__ in, T* __restrict__ out, size_t rows, size_t D) {
    constexpr int RPB = SB / TPR;
    const size_t row = (size_t)blockIdx.x * RPB + threadIdx.x / TPR;
    const unsigned t = threadIdx.x % TPR;
    const bool live = row < rows;
    const T* src = in + (live ? row : 0) * D;
    T* dst = out + (live ? row : 0) * D;
    __shared__ float red[SB / WAVE];
    AVec<T, VEC> keep[FITS ? NREG : 1];
    const size_t step = (size_t)TPR * VEC;
    auto load = [&](size_t i) {
        AVec<T, VEC> v;
        if constexpr (VEC > 1) v = *(const AVec<T, VEC>*)(src + i);
        else v.v[0] = src[i];
        return v;
    };
    auto store = [&](size_t i, const AVec<T, VEC>& o) {
        if constexpr (VEC > 1) *(AVec<T, VEC>*)(dst + i) = o;
        else dst[i] = o.v[0];
    };

    float m = -INFINITY;
    if (live) {
        if constexpr (FITS) {
#pragma unroll
            for (int k = 0; k < NREG; ++k) {
                const size_t i = (size_t)t * VEC + k * step;
                if (i < D) {
                    keep[k] = load(i);
#pragma unroll
                    for (int e = 0; e < VEC; ++e) { float x = SM<T>::ld(keep[k].v[e]); m = x > m ? x : m; }
                }
            }
        } else {
            for (size_t i = (size_t)t * VEC; i < D; i += step) {
                const AVec<T, VEC> v = load(i);
#pragma unroll
                for (int e = 0; e < VEC; ++e) { float x = SM<T>::ld(v.v[e]); m = x > m ? x : m; }
            }
        }
    }
    m = wave_max<(TPR < WAVE ? TPR : WAVE)>(m);
    if constexpr (TPR > WAVE) {
        if (threadIdx.x % WAVE == 0) red[threadIdx.x / WAVE] = m;
        __syncthreads();
        m = red[0];
#pragma unroll
        for (int w = 1; w < SB / WAVE; ++w) m = red[w] > m ? red[w] : m;
        __syncthreads();
    }

    float s = 0.0f;
    if (live) {
        if constexpr (FITS) {
#pragma unroll
            for (int k = 0; k < NREG; ++k) {
                const size_t i = (size_t)t * VEC + k * step;
                if (i < D) {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        const float ev = SM<T>::shifted(SM<T>::ld(keep[k].v[e]), m);
                        SM<T>::keep(keep[k].v[e], ev);
                        s += ev;
                    }
                }
            }
        } else {
            for (size_t i = (size_t)t * VEC; i < D; i += step) {
                const AVec<T, VEC> v = load(i);
#pragma unroll
                for (int e = 0; e < VEC; ++e) s += SM<T>::shifted(SM<T>::ld(v.v[e]), m);
            }
        }
    }
    s = wave_sum<(TPR < WAVE ? TPR : WAVE)>(s);
    if constexpr (TPR > WAVE) {
        if (threadIdx.x % WAVE == 0) red[threadIdx.x / WAVE] = s;
        __syncthreads();
        s = red[0];
#pragma unroll
        for (int w = 1; w < SB / WAVE; ++w) s += red[w];
    }
    s = m_exp(-INFINITY - m) + s;      // 0, or NaN when no element beat -inf

    if (!live) return;
    if constexpr (FITS) {
#pragma unroll
        for (int k = 0; k < NREG; ++k) {
            const size_t i = (size_t)t * VEC + k * step;
            if (i < D) {
                AVec<T, VEC> o;
#pragma unroll
                for (int e = 0; e < VEC; ++e) o.v[e] = SM<T>::fin(SM<T>::ld(keep[k].v[e]), s);
                store(i, o);
            }
        }
    } else {
        for (size_t i = (size_t)t * VEC; i < D; i += step) {
            const AVec<T, VEC> v = load(i);
            AVec<T, VEC> o;
#pragma unroll
            for (int e = 0; e < VEC; ++e) o.v[e] = SM<T>::fin(SM<T>::shifted(SM<T>::ld(v.v[e]), m), s);
            store(i, o);
        }
    }
}

// The same for bf16 / f16 with exp(x - m) taken from the dtype's table of exp (lut16.hpp): the term the kernel above
// computes is round(exp(round(x - m))), a function of one 16-bit value, i.e. an entry of the table that hip_exp_<T> is
// served from - the same bits.  The arithmetic form is bound by the bit-exact expf (28 % of HBM peak on [8192,8192]).
// Here one 1024-thread block per CU copies the 128 KB table into LDS once, and then every WAVE works through rows of its
// own, with no barrier: lane l stands for threads l, 64 + l, ... of the kernel above (VW of them: that kernel's block of
// 64 * VW threads), holds their elements, adds their terms in their order into VW separate sums, folds each across the
// wave as that kernel's waves do and adds the VW results in wave order - the same additions, the same bits.  The maximum
// takes no part in this: no NaN ever enters it, and max over numbers does not depend on the order.  The 16 waves of a CU
// drift apart, so loads, lookups and stores of different rows overlap; PF also fetches a wave's next row before it works
// on the current one.  The row must fit the registers (D <= 64 * VW * VEC * NREG).
template <class T> struct SMCode;
template <> struct SMCode<bf16_t> { static __device__ uint32_t of(float v) { return f2bf(v).bits; } };
template <> struct SMCode<f16_t> { static __device__ uint32_t of(float v) { return f2h(v).bits; } };
template <class T, int TPR, int VW, int VEC, int NREG>
struct LutRow {
    AVec<T, VEC> v[VW][NREG];
    static __device__ size_t at(int w, int k, unsigned t) { return (size_t)(w * TPR + t) * VEC + (size_t)k * (VW * TPR * VEC); }
    __device__ void load(const T* __restrict__ src, unsigned t, size_t D) {
#pragma unroll
        for (int w = 0; w < VW; ++w)
#pragma unroll
            for (int k = 0; k < NREG; ++k)
                if (at(w, k, t) < D) v[w][k] = *(const AVec<T, VEC>*)(src + at(w, k, t));
    }
};
// TPR < 64 (short rows, VW = 1): 64 / TPR rows per wave, a group of TPR lanes each, as in the kernel above.
template <class T, int TPR, int VW, int VEC, int NREG, bool PF, int BLK>
__global__ __launch_bounds__(BLK) void softmax_row_lut_kernel(const uint16_t* __restrict__ table, const T* __restrict__ in, T* __restrict__ out,
                                                              size_t rows, size_t D) {
    static_assert(TPR == WAVE || VW == 1, "several waves' worth of threads only for whole-wave rows");
    extern __shared__ __attribute__((aligned(16))) uint16_t lut[];
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    for (int i = threadIdx.x; i < 65536 * 2 / 16; i += BLK) ((u4*)lut)[i] = ((const u4*)table)[i];
    __syncthreads();
    constexpr int RPW = WAVE / TPR;
    const unsigned lane = threadIdx.x % WAVE, t = lane % TPR;
    const size_t stride = (size_t)gridDim.x * (BLK / WAVE) * RPW;
    size_t row = ((size_t)blockIdx.x * (BLK / WAVE) + threadIdx.x / WAVE) * RPW + lane / TPR;
    typedef LutRow<T, TPR, VW, VEC, NREG> Row;
    Row cur, nxt;
    if (row < rows) cur.load(in + row * D, t, D);
    // a wave leaves the loop when its first row is past the end; the groups behind it are then past it too
    for (; row - lane / TPR < rows; row += stride) {
        const bool live = row < rows;
        if (PF && row + stride < rows) nxt.load(in + (row + stride) * D, t, D);
        float m = -INFINITY;
        if (live) {
#pragma unroll
            for (int w = 0; w < VW; ++w)
#pragma unroll
                for (int k = 0; k < NREG; ++k)
                    if (Row::at(w, k, t) < D) {
#pragma unroll
                        for (int e = 0; e < VEC; ++e) { float x = SM<T>::ld(cur.v[w][k].v[e]); m = x > m ? x : m; }
                    }
        }
        m = wave_max<TPR>(m);
        float s = 0.0f;
#pragma unroll
        for (int w = 0; w < VW; ++w) {
            float sw = 0.0f;
            if (live) {
#pragma unroll
                for (int k = 0; k < NREG; ++k)
                    if (Row::at(w, k, t) < D) {
#pragma unroll
                        for (int e = 0; e < VEC; ++e) {
                            T en;
                            en.bits = lut[SMCode<T>::of(SM<T>::ld(cur.v[w][k].v[e]) - m)];
                            cur.v[w][k].v[e] = en;          // the term is a 16-bit value: it stays where x was
                            sw += SM<T>::ld(en);
                        }
                    }
            }
            sw = wave_sum<TPR>(sw);
            s = w == 0 ? sw : s + sw;
        }
        s = m_exp(-INFINITY - m) + s;
        if (live) {
            T* dst = out + row * D;
#pragma unroll
            for (int w = 0; w < VW; ++w)
#pragma unroll
                for (int k = 0; k < NREG; ++k)
                    if (Row::at(w, k, t) < D) {
                        AVec<T, VEC> o;
#pragma unroll
                        for (int e = 0; e < VEC; ++e) o.v[e] = SM<T>::fin(SM<T>::ld(cur.v[w][k].v[e]), s);
                        *(AVec<T, VEC>*)(dst + Row::at(w, k, t)) = o;
                    }
        }
        if (PF) cur = nxt;
        else if (row + stride < rows) cur.load(in + (row + stride) * D, t, D);
    }
}

// [pre, D, post] contiguous, post > 1: one thread per (pre, post) column
template <class T>
__global__ __launch_bounds__(SB) void softmax_col_kernel(const T* __restrict__ in, T* __restrict__ out, size_t slices, size_t D,
                                                         size_t post) {
    size_t s_id = (size_t)blockIdx.x * SB + threadIdx.x;
    if (s_id >= slices) return;
    size_t pre_idx = s_id / post, post_idx = s_id % post;
    const T* src = in + pre_idx * D * post + post_idx;
    T* dst = out + pre_idx * D * post + post_idx;
    float m = -INFINITY;
    for (size_t i = 0; i < D; ++i) { float x = SM<T>::ld(src[i * post]); m = x > m ? x : m; }
    float s = 0.0f;
    for (size_t i = 0; i < D; ++i) s += SM<T>::shifted(SM<T>::ld(src[i * post]), m);
    s = m_exp(-INFINITY - m) + s;
    for (size_t i = 0; i < D; ++i) dst[i * post] = SM<T>::fin(SM<T>::shifted(SM<T>::ld(src[i * post]), m), s);
}

// [pre, D, post] contiguous, long D: a block of NW waves shares 64*VEC columns and splits D among its
// waves; the per-wave maxima and sums meet in LDS (in wave order).  Three passes over the block's slab.
template <class T, int VEC, int NW>
__global__ __launch_bounds__(WAVE * NW) void softmax_col_split_kernel(const T* __restrict__ in, T* __restrict__ out, size_t D,
                                                                       size_t post, uint32_t cv, FastDiv div_jb) {
    const int lane = threadIdx.x % WAVE, w = threadIdx.x / WAVE;
    uint32_t pre_idx, jb;
    fd_divmod(blockIdx.x, div_jb, pre_idx, jb);
    const uint32_t j = jb * WAVE + lane;           // column vector inside the slab
    const bool live = j < cv;
    const size_t slice = (D + NW - 1) / NW;
    const size_t l0 = (size_t)w * slice < D ? (size_t)w * slice : D, l1 = l0 + slice < D ? l0 + slice : D;
    const T* src = in + (size_t)pre_idx * D * post + (size_t)j * VEC;
    T* dst = out + (size_t)pre_idx * D * post + (size_t)j * VEC;
    __shared__ float red[NW][VEC][WAVE];
    auto load = [&](size_t l) {
        AVec<T, VEC> v;
        if constexpr (VEC > 1) v = *(const AVec<T, VEC>*)(src + l * post);
        else v.v[0] = src[l * post];
        return v;
    };
    auto combine = [&](float (&a)[VEC], bool is_max) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) red[w][e][lane] = a[e];
        __syncthreads();
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            float t = red[0][e][lane];
#pragma unroll
            for (int k = 1; k < NW; ++k) t = is_max ? (red[k][e][lane] > t ? red[k][e][lane] : t) : t + red[k][e][lane];
            a[e] = t;
        }
        __syncthreads();
    };
    // 8 KB of loads in flight per wave (a wave's row is one or a few cache lines: taken one at a time, every row costs
    // a memory latency, and with few bytes per row the 2048 waves of a [8192,8192] launch cannot cover the latency
    // between them); the rows are still folded in ascending order
    constexpr int ROW_BYTES = WAVE * VEC * (int)sizeof(T);
    constexpr int U = 8192 / ROW_BYTES < 8 ? 8 : (8192 / ROW_BYTES > 32 ? 32 : 8192 / ROW_BYTES);
    auto sweep = [&](auto&& each) {
        size_t l = l0;
        for (; l + U <= l1; l += U) {
            AVec<T, VEC> v[U];
#pragma unroll
            for (int k = 0; k < U; ++k) v[k] = load(l + k);
#pragma unroll
            for (int k = 0; k < U; ++k) each(l + k, v[k]);
        }
        for (; l < l1; ++l) each(l, load(l));
    };
    float m[VEC], s[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) { m[e] = -INFINITY; s[e] = 0.0f; }
    if (live)
        sweep([&](size_t, const AVec<T, VEC>& v) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) { float x = SM<T>::ld(v.v[e]); m[e] = x > m[e] ? x : m[e]; }
        });
    combine(m, true);
    if (live)
        sweep([&](size_t, const AVec<T, VEC>& v) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) s[e] += SM<T>::shifted(SM<T>::ld(v.v[e]), m[e]);
        });
    combine(s, false);
    if (!live) return;
#pragma unroll
    for (int e = 0; e < VEC; ++e) s[e] = m_exp(-INFINITY - m[e]) + s[e];
    sweep([&](size_t l, const AVec<T, VEC>& v) {
        AVec<T, VEC> o;
#pragma unroll
        for (int e = 0; e < VEC; ++e) o.v[e] = SM<T>::fin(SM<T>::shifted(SM<T>::ld(v.v[e]), m[e]), s[e]);
        if constexpr (VEC > 1) *(AVec<T, VEC>*)(dst + l * post) = o;
        else dst[l * post] = o.v[0];
    });
}

// [pre, D, post] contiguous, long D and few columns per CU (a [8192,8192] matrix along dim 0: one block per 64 column
// vectors would be 32 blocks): the rows are cut into `groups` groups and a thread owns one column vector for one group's
// rows, consecutive threads on consecutive vectors (a block reads 4 KB of a row at a time), eight rows in flight; three
// launches that each read the rows once -
//   PHASE 0: the maximum of every column over the group's rows                      -> part[pre][group][post]
//   PHASE 1: the group's sum of exp(x - m), m = the column's maximum                 -> part[pre][group][post]
//   PHASE 2: out = exp(x - m) / s
// with softmax_col_fold_kernel between them, which folds the groups' values of a column in group order into
// m[pre][post] (exact) and s[pre][post] = exp(-inf - m) + sum.
// LUT (bf16 / f16): exp(x - m) is the entry of the dtype's table of exp, held in LDS, for the code of the rounded
// difference - the bits SM<T>::shifted computes (see softmax_row_lut_kernel).
template <class T, int VEC, int PHASE, bool STREAM, bool LUT>
__device__ __forceinline__ void softmax_col_groups_body(uint32_t vblock, uint32_t tid, const uint16_t* lut, const T* __restrict__ in,
                                                        T* __restrict__ out, float* __restrict__ part, const float* __restrict__ cmax,
                                                        const float* __restrict__ csum, size_t D, size_t post, uint32_t cv, uint32_t slabs,
                                                        uint32_t groups, uint32_t rows_per_group) {
    constexpr int U = 8;
    const uint32_t slab = vblock % slabs, group = (vblock / slabs) % groups, pre_idx = vblock / (slabs * groups);
    const uint32_t j = slab * 256 + tid;                   // column vector
    if (j >= cv) return;
    auto term = [&](T x, float mx) -> float {
        if constexpr (LUT) {
            T en;
            en.bits = lut[SMCode<T>::of(SM<T>::ld(x) - mx)];
            return SM<T>::ld(en);
        } else {
            return SM<T>::shifted(SM<T>::ld(x), mx);
        }
    };
    const size_t l0 = (size_t)group * rows_per_group < D ? (size_t)group * rows_per_group : D;
    const size_t l1 = l0 + rows_per_group < D ? l0 + rows_per_group : D;
    const T* src = in + (size_t)pre_idx * D * post + (size_t)j * VEC;
    T* dst = out + (size_t)pre_idx * D * post + (size_t)j * VEC;
    float* mine = part + ((size_t)pre_idx * groups + group) * post + (size_t)j * VEC;
    const size_t col = (size_t)pre_idx * post + (size_t)j * VEC;
    auto sweep = [&](auto&& each) {
        size_t l = l0;
        for (; l + U <= l1; l += U) {
            AVec<T, VEC> v[U];
#pragma unroll
            for (int k = 0; k < U; ++k) v[k] = ld_vec<STREAM>((const AVec<T, VEC>*)(src + (l + k) * post));
#pragma unroll
            for (int k = 0; k < U; ++k) each(l + k, v[k]);
        }
        for (; l < l1; ++l) each(l, ld_vec<STREAM>((const AVec<T, VEC>*)(src + l * post)));
    };
    float m[VEC], s[VEC];
    if constexpr (PHASE == 0) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) m[e] = -INFINITY;
        sweep([&](size_t, const AVec<T, VEC>& v) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) { float x = SM<T>::ld(v.v[e]); m[e] = x > m[e] ? x : m[e]; }
        });
        AVec<float, VEC> r;
#pragma unroll
        for (int e = 0; e < VEC; ++e) r.v[e] = m[e];
        *(AVec<float, VEC>*)mine = r;
    } else {
        const AVec<float, VEC> mv = *(const AVec<float, VEC>*)(cmax + col);
#pragma unroll
        for (int e = 0; e < VEC; ++e) m[e] = mv.v[e];
        if constexpr (PHASE == 1) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) s[e] = 0.0f;
            sweep([&](size_t, const AVec<T, VEC>& v) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) s[e] += term(v.v[e], m[e]);
            });
            AVec<float, VEC> r;
#pragma unroll
            for (int e = 0; e < VEC; ++e) r.v[e] = s[e];
            *(AVec<float, VEC>*)mine = r;
        } else {
            const AVec<float, VEC> sv = *(const AVec<float, VEC>*)(csum + col);
#pragma unroll
            for (int e = 0; e < VEC; ++e) s[e] = sv.v[e];
            sweep([&](size_t l, const AVec<T, VEC>& v) {
                AVec<T, VEC> o;
#pragma unroll
                for (int e = 0; e < VEC; ++e) o.v[e] = SM<T>::fin(term(v.v[e], m[e]), s[e]);
                st_vec<STREAM>((AVec<T, VEC>*)(dst + l * post), o);
            });
        }
    }
}
template <class T, int VEC, int PHASE, bool STREAM>
__global__ __launch_bounds__(256) void softmax_col_groups_kernel(const T* __restrict__ in, T* __restrict__ out, float* __restrict__ part,
                                                                 const float* __restrict__ cmax, const float* __restrict__ csum, size_t D,
                                                                 size_t post, uint32_t cv, uint32_t slabs, uint32_t groups,
                                                                 uint32_t rows_per_group) {
    softmax_col_groups_body<T, VEC, PHASE, STREAM, false>(blockIdx.x, threadIdx.x, nullptr, in, out, part, cmax, csum, D, post, cv, slabs, groups,
                                                          rows_per_group);
}
// The same work by one persistent 1024-thread block per CU that holds the table: every quarter of the block is one block
// of the kernel above after the other (no barrier between them: a thread's columns are its own).
template <class T, int VEC, int PHASE, bool STREAM>
__global__ __launch_bounds__(1024) void softmax_col_groups_lut_kernel(const uint16_t* __restrict__ table, uint32_t vblocks, const T* __restrict__ in,
                                                                      T* __restrict__ out, float* __restrict__ part, const float* __restrict__ cmax,
                                                                      const float* __restrict__ csum, size_t D, size_t post, uint32_t cv,
                                                                      uint32_t slabs, uint32_t groups, uint32_t rows_per_group) {
    extern __shared__ __attribute__((aligned(16))) uint16_t lut[];
    typedef uint32_t u4 __attribute__((ext_vector_type(4)));
    for (int i = threadIdx.x; i < 65536 * 2 / 16; i += 1024) ((u4*)lut)[i] = ((const u4*)table)[i];
    __syncthreads();
    for (uint32_t vb = blockIdx.x * 4 + threadIdx.x / 256; vb < vblocks; vb += gridDim.x * 4)
        softmax_col_groups_body<T, VEC, PHASE, STREAM, true>(vb, threadIdx.x % 256, lut, in, out, part, cmax, csum, D, post, cv, slabs, groups,
                                                             rows_per_group);
}

// SUM ? s = exp(-inf - m) + part[0] + part[1] + ... : m = max(part[0], part[1], ...) for every column.  A block is 64
// columns (the lanes) by 16 waves; wave w folds the w-th sixteenth of the groups in ascending order, eight loads in
// flight, and the sixteen results meet in LDS in wave order.
template <bool SUM>
__global__ __launch_bounds__(1024) void softmax_col_fold_kernel(const float* __restrict__ part, const float* __restrict__ cmax, float* __restrict__ res,
                                                                size_t post, size_t cols, uint32_t groups) {
    constexpr int NW = 16;
    const int lane = threadIdx.x % WAVE, w = threadIdx.x / WAVE;
    const size_t c = (size_t)blockIdx.x * WAVE + lane;
    const bool live = c < cols;
    __shared__ float red[NW][WAVE];
    const uint32_t per = (groups + NW - 1) / NW;
    const uint32_t g0 = w * per < groups ? w * per : groups, g1 = g0 + per < groups ? g0 + per : groups;
    float t = SUM ? 0.0f : -INFINITY;
    if (live && g0 < g1) {
        const size_t pre_idx = c / post, j = c - pre_idx * post;
        const float* p = part + pre_idx * groups * post + j;
        t = p[(size_t)g0 * post];
        uint32_t g = g0 + 1;
        for (; g + 8 <= g1; g += 8) {
            float v[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) v[k] = p[(size_t)(g + k) * post];
#pragma unroll
            for (int k = 0; k < 8; ++k) t = SUM ? t + v[k] : (v[k] > t ? v[k] : t);
        }
        for (; g < g1; ++g) { const float v = p[(size_t)g * post]; t = SUM ? t + v : (v > t ? v : t); }
    }
    red[w][lane] = t;
    __syncthreads();
    if (w != 0 || !live) return;
    t = red[0][lane];
#pragma unroll
    for (int k = 1; k < NW; ++k) {
        if (k * per >= groups) break;            // (waves without groups hold the neutral value, but 0 + (-0) would lose a sign)
        t = SUM ? t + red[k][lane] : (red[k][lane] > t ? red[k][lane] : t);
    }
    res[c] = SUM ? m_exp(-INFINITY - cmax[c]) + t : t;
}

struct SoftmaxStrided {
    int nd, dim;
    uint32_t dims[MAXD];
    int64_t strides[MAXD];
};

template <class T>
__global__ __launch_bounds__(SB) void softmax_strided_kernel(SoftmaxStrided sp, const T* __restrict__ in, T* __restrict__ out,
                                                             size_t slices, size_t D, size_t post) {
    size_t s_id = (size_t)blockIdx.x * SB + threadIdx.x;
    if (s_id >= slices) return;
    size_t pre_idx = s_id / post, post_idx = s_id % post;
    int64_t base = 0;
    {
        size_t rem = pre_idx;
        for (int d = 0; d < sp.dim; ++d) { base += (int64_t)(rem % sp.dims[d]) * sp.strides[d]; rem /= sp.dims[d]; }
        rem = post_idx;
        for (int d = sp.nd - 1; d > sp.dim; --d) { base += (int64_t)(rem % sp.dims[d]) * sp.strides[d]; rem /= sp.dims[d]; }
    }
    const int64_t st = sp.strides[sp.dim];
    T* dst = out + pre_idx * D * post + post_idx;
    float m = -INFINITY;
    for (size_t i = 0; i < D; ++i) { float x = SM<T>::ld(in[base + (int64_t)i * st]); m = x > m ? x : m; }
    float s = 0.0f;
    for (size_t i = 0; i < D; ++i) s += SM<T>::shifted(SM<T>::ld(in[base + (int64_t)i * st]), m);
    s = m_exp(-INFINITY - m) + s;
    for (size_t i = 0; i < D; ++i) dst[i * post] = SM<T>::fin(SM<T>::shifted(SM<T>::ld(in[base + (int64_t)i * st]), m), s);
}

template <class T>
void softmax(size_t num_els, size_t nd, size_t dim_arg, const size_t* md, const T* in, T* out) {
    if (!md || !in || !out) return;       // the reference returns silently (:66-68)
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
    const T* src = in + offset;
    if (cont && post == 1) {
        constexpr int VEC = 16 / sizeof(T);
        const bool vec = D % VEC == 0 && ((uintptr_t)src % 16) == 0 && ((uintptr_t)out % 16) == 0;
        if (slices >= (1ull << 31)) { set_status(ERR_TOO_LARGE, "softmax: 2^31 or more rows"); return; }
        if constexpr (sizeof(T) == 2) {
            // a large 16-bit call whose rows fit the registers: exp from the table, one persistent block per CU (filling
            // the tables costs every block about 3 us: below 2^22 elements the arithmetic kernel is as fast)
            if (vec && slices * D >= (1u << 22) && D <= (size_t)SB * VEC * 4) {
                const uint16_t* table = std::is_same<T, bf16_t>::value ? lut16_exp_bf16() : lut16_exp_f16();
                static int cus[16] = {0};
                int dev = 0;
                if (table && hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 16) {
                    if (!cus[dev]) {
                        hipDeviceProp_t prop;
                        cus[dev] = hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
                    }
                    constexpr int LUT_LDS = 65536 * 2;
                    auto launch = [&](auto kern, int blk, int tpr) {
                        static bool allowed[16] = {false};
                        if (!allowed[dev]) {
                            if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, LUT_LDS) != hipSuccess) { (void)hipGetLastError(); return false; }
                            allowed[dev] = true;
                        }
                        const unsigned blocks = (unsigned)std::min<size_t>((size_t)cus[dev], cdiv(slices, (size_t)(blk / tpr)));
                        hipLaunchKernelGGL(kern, dim3(blocks), dim3(blk), LUT_LDS, stream(), table, src, out, slices, D);
                        MXH_LAUNCH_CHECK("softmax_row_lut");
                        return true;
                    };
                    // lanes per row, vectors per lane and waves' worth of lanes follow the arithmetic kernels below
                    constexpr int WV = SB / WAVE, NW = 2048 / (WAVE * VEC);
                    if (D <= 8 * VEC    ? launch(softmax_row_lut_kernel<T, 8, 1, VEC, 1, true, 1024>, 1024, 8)
                        : D <= 16 * VEC ? launch(softmax_row_lut_kernel<T, 16, 1, VEC, 1, true, 1024>, 1024, 16)
                        : D <= 32 * VEC ? launch(softmax_row_lut_kernel<T, 32, 1, VEC, 1, true, 1024>, 1024, 32)
                        : D <= 2048     ? launch(softmax_row_lut_kernel<T, WAVE, 1, VEC, NW, true, 1024>, 1024, WAVE)
                        : D <= (size_t)SB * VEC * 2 ? launch(softmax_row_lut_kernel<T, WAVE, WV, VEC, 2, false, 1024>, 1024, WAVE)
                                                    : launch(softmax_row_lut_kernel<T, WAVE, WV, VEC, 4, false, 512>, 512, WAVE))
                        return;
                }
            }
        }
        if (D <= 2048) {
            unsigned blocks = cdiv(slices, SB / WAVE);
            // short rows: 8, 16 or 32 lanes each, so that a wave holds several
            auto narrow = [&](auto kern, int tpr) { hipLaunchKernelGGL(kern, dim3((unsigned)cdiv(slices, (size_t)(SB / tpr))), dim3(SB), 0, stream(), src, out, slices, D); };
            if (vec && D <= 8 * VEC) narrow(softmax_row_kernel<T, 8, VEC, 1, true>, 8);
            else if (vec && D <= 16 * VEC) narrow(softmax_row_kernel<T, 16, VEC, 1, true>, 16);
            else if (vec && D <= 32 * VEC) narrow(softmax_row_kernel<T, 32, VEC, 1, true>, 32);
            else if (vec) hipLaunchKernelGGL((softmax_row_kernel<T, WAVE, VEC, 2048 / (WAVE * VEC), true>), dim3(blocks), dim3(SB), 0, stream(), src, out, slices, D);
            else if (D <= WAVE * 8) hipLaunchKernelGGL((softmax_row_kernel<T, WAVE, 1, 8, true>), dim3(blocks), dim3(SB), 0, stream(), src, out, slices, D);
            else hipLaunchKernelGGL((softmax_row_kernel<T, WAVE, 1, 8, false>), dim3(blocks), dim3(SB), 0, stream(), src, out, slices, D);
        } else {
            if (vec && D <= (size_t)SB * VEC * 8) hipLaunchKernelGGL((softmax_row_kernel<T, SB, VEC, 8, true>), dim3((unsigned)slices), dim3(SB), 0, stream(), src, out, slices, D);
            else if (vec) hipLaunchKernelGGL((softmax_row_kernel<T, SB, VEC, 8, false>), dim3((unsigned)slices), dim3(SB), 0, stream(), src, out, slices, D);
            else hipLaunchKernelGGL((softmax_row_kernel<T, SB, 1, 8, false>), dim3((unsigned)slices), dim3(SB), 0, stream(), src, out, slices, D);
        }
        MXH_LAUNCH_CHECK("softmax_row");
        return;
    }
    if (slices >= (1ull << 38)) { set_status(ERR_TOO_LARGE, "softmax: 2^38 or more slices"); return; }
    if (cont && D >= 64 && pre * cdiv(post, (size_t)WAVE) < (1ull << 31) && post < (1ull << 31)) {
        // long columns: blocks of 16 waves; narrow vectors when wide ones would leave CUs without a block
        constexpr int VEC = 16 / sizeof(T), NW = 16;
        const bool vec_ok = post % VEC == 0 && ((uintptr_t)src % 16) == 0 && ((uintptr_t)out % 16) == 0;
        const size_t blocks_v = pre * cdiv(post / VEC, (size_t)WAVE);
        // few columns per CU and long ones: the rows in groups, three launches (see softmax_col_groups_kernel)
        if (vec_ok && blocks_v < 1024 && D >= 1024 && pre * post < (1ull << 31)) {
            const uint32_t cv = (uint32_t)(post / VEC), slabs = (uint32_t)cdiv(cv, (size_t)256);
            uint32_t groups = (uint32_t)std::min<size_t>(std::min<size_t>(cdiv((size_t)2048, pre * slabs), D / 16), 256);
            const uint32_t rpg = (uint32_t)cdiv(D, (size_t)groups);
            groups = (uint32_t)cdiv(D, (size_t)rpg);
            const size_t part_n = pre * groups * post, cols = pre * post;
            float* part = (float*)scratch((part_n + 2 * cols) * sizeof(float));
            if (!part) return;
            float *cm = part + part_n, *cs = cm + cols;
            const dim3 grid((unsigned)(pre * slabs * groups)), block(256), fold((unsigned)cdiv(cols, (size_t)WAVE)), fold_block(1024);
            const bool big = ew_stream_bytes() != 0 && num_els * sizeof(T) >= ew_stream_bytes();
#define MXH_SM_PHASE(P)                                                                                                                   \
    if (big) hipLaunchKernelGGL((softmax_col_groups_kernel<T, VEC, P, true>), grid, block, 0, stream(), src, out, part, cm, cs, D, post, cv, slabs, groups, rpg); \
    else hipLaunchKernelGGL((softmax_col_groups_kernel<T, VEC, P, false>), grid, block, 0, stream(), src, out, part, cm, cs, D, post, cv, slabs, groups, rpg)
            // 16-bit, 2^22 elements or more: the two phases with exp in them by table, one persistent block per CU
            const uint16_t* table = nullptr;
            int dev = 0, cus = 0;
            if constexpr (sizeof(T) == 2) {
                if (num_els >= (1u << 22) && hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < 16) {
                    table = std::is_same<T, bf16_t>::value ? lut16_exp_bf16() : lut16_exp_f16();
                    static int cu_count[16] = {0};
                    if (!cu_count[dev]) {
                        hipDeviceProp_t prop;
                        cu_count[dev] = hipGetDeviceProperties(&prop, dev) == hipSuccess && prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
                    }
                    cus = cu_count[dev];
                }
            }
            auto by_table = [&](auto kern) {
                static bool allowed[16] = {false};
                if (!table) return false;
                if (!allowed[dev]) {
                    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 65536 * 2) != hipSuccess) { (void)hipGetLastError(); return false; }
                    allowed[dev] = true;
                }
                const uint32_t vblocks = grid.x;
                hipLaunchKernelGGL(kern, dim3(std::min<unsigned>((unsigned)cus, (unsigned)cdiv((size_t)vblocks, (size_t)4))), dim3(1024), 65536 * 2, stream(), table,
                                   vblocks, src, out, part, (const float*)cm, (const float*)cs, D, post, cv, slabs, groups, rpg);
                return true;
            };
            bool done = false;
            MXH_SM_PHASE(0);
            hipLaunchKernelGGL((softmax_col_fold_kernel<false>), fold, fold_block, 0, stream(), part, (const float*)nullptr, cm, post, cols, groups);
            if constexpr (sizeof(T) == 2) done = big ? by_table(softmax_col_groups_lut_kernel<T, VEC, 1, true>) : by_table(softmax_col_groups_lut_kernel<T, VEC, 1, false>);
            if (!done) { MXH_SM_PHASE(1); }
            hipLaunchKernelGGL((softmax_col_fold_kernel<true>), fold, fold_block, 0, stream(), part, cm, cs, post, cols, groups);
            done = false;
            if constexpr (sizeof(T) == 2) done = big ? by_table(softmax_col_groups_lut_kernel<T, VEC, 2, true>) : by_table(softmax_col_groups_lut_kernel<T, VEC, 2, false>);
            if (!done) { MXH_SM_PHASE(2); }
#undef MXH_SM_PHASE
            MXH_LAUNCH_CHECK("softmax_col_groups");
            return;
        }
        if (vec_ok && blocks_v >= 256) {
            uint32_t cv = (uint32_t)(post / VEC), jb = (uint32_t)cdiv(cv, (size_t)WAVE);
            hipLaunchKernelGGL((softmax_col_split_kernel<T, VEC, NW>), dim3((unsigned)(pre * jb)), dim3(WAVE * NW), 0, stream(), src, out, D, post, cv, make_fastdiv(jb));
        } else {
            uint32_t cv = (uint32_t)post, jb = (uint32_t)cdiv(cv, (size_t)WAVE);
            hipLaunchKernelGGL((softmax_col_split_kernel<T, 1, NW>), dim3((unsigned)(pre * jb)), dim3(WAVE * NW), 0, stream(), src, out, D, post, cv, make_fastdiv(jb));
        }
        MXH_LAUNCH_CHECK("softmax_col_split");
        return;
    }
    if (cont) {
        hipLaunchKernelGGL(softmax_col_kernel<T>, dim3(cdiv(slices, SB)), dim3(SB), 0, stream(), src, out, slices, D, post);
        MXH_LAUNCH_CHECK("softmax_col");
        return;
    }
    // A large strided input with at most one leading dim of more than one element: the reference's walk of the leading
    // dims (dim 0 fastest, see softmax_strided_kernel) is then the ordinary one, and the call is the contiguous softmax
    // of a logical-order copy, which the elementwise identity makes by the same index rule ([4096,4096] viewed
    // transposed: 2800 / 4300 us with a thread per slice).  Not while a capture is open (the scratch block cannot grow).
    {
        size_t leading = 0;
        for (size_t d = 0; d < dim; ++d) leading += dims[d] > 1;
        if (leading <= 1 && num_els >= (1u << 18) && num_els < (1ull << 31) && nd <= 64 && !capture_open()) {
            T* tmp = (T*)scratch(num_els * sizeof(T), 1);
            if (!tmp) return;
            size_t cmd[2 * 64 + 1];
            for (size_t d = 0; d < nd; ++d) cmd[d] = dims[d];
            contiguous_strides(nd, dims, cmd + nd);
            cmd[2 * nd] = 0;
            const size_t* ins[1] = {strides};
            const void* inp[1] = {src};
            ew_launch<OpIdentity<T>>(num_els, nd, dims, cmd + nd, ins, tmp, inp, OpIdentity<T>{});
            softmax<T>(num_els, nd, dim, cmd, tmp, out);
            return;
        }
    }
    if (nd > (size_t)MAXD) { set_status(ERR_UNSUPPORTED, "softmax: strided input of rank above 8"); return; }
    SoftmaxStrided sp;
    sp.nd = (int)nd; sp.dim = (int)dim;
    for (int d = 0; d < MAXD; ++d) {
        sp.dims[d] = d < (int)nd ? (uint32_t)dims[d] : 1;
        sp.strides[d] = d < (int)nd ? (int64_t)strides[d] : 0;
    }
    hipLaunchKernelGGL(softmax_strided_kernel<T>, dim3(cdiv(slices, SB)), dim3(SB), 0, stream(), sp, src, out, slices, D, post);
    MXH_LAUNCH_CHECK("softmax_strided");
}

}  // namespace mxh

using namespace mxh;

extern "C" void hip_softmax_f32(size_t num_els, size_t num_dims, size_t dim, const size_t* md, const float* in, float* out) { MXH_API;
    softmax<float>(num_els, num_dims, dim, md, in, out);
}
extern "C" void hip_softmax_f16(size_t num_els, size_t num_dims, size_t dim, const size_t* md, const f16_t* in, f16_t* out) { MXH_API;
    softmax<f16_t>(num_els, num_dims, dim, md, in, out);
}
extern "C" void hip_softmax_bf16(size_t num_els, size_t num_dims, size_t dim, const size_t* md, const bf16_t* in, bf16_t* out) { MXH_API;
    softmax<bf16_t>(num_els, num_dims, dim, md, in, out);
}
