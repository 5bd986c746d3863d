// Reducers, the 16-bit rounding helpers, the wave64 butterfly and the row-reduce kernel: shared by the
// reductions and by the interpreter of recorded programs.
#pragma once
#include <cfloat>

#include "elementwise.hpp"
#include "mxh.hpp"

namespace mxh {

// ---- reducers -------------------------------------------------------------------------------
struct RSum {
    static __device__ float init(bool) { return 0.0f; }
    static __device__ float op(float a, float b) { return a + b; }
};
// `if val > out { val } else { out }` from f32::MIN: NaNs never win, −inf does not beat the seed.
struct RMax {
    static __device__ float init(bool is_bf16) { return is_bf16 ? -INFINITY : -FLT_MAX; }   // bf16(f32::MIN) is −inf
    static __device__ float op(float a, float b) { return b > a ? b : a; }
};
struct RMin {
    static __device__ float init(bool is_bf16) { return is_bf16 ? INFINITY : FLT_MAX; }
    static __device__ float op(float a, float b) { return b < a ? b : a; }
};

template <class T> struct IO;
template <> struct IO<float> {
    static constexpr bool is_bf16 = false;
    static __device__ float ld(float v) { return v; }
    // div != 0: the mean's single division at the end (reduction.rs:264-268)
    static __device__ float fin(float acc, float div) { return div != 0.0f ? acc / div : acc; }
};
template <> struct IO<bf16_t> {
    static constexpr bool is_bf16 = true;
    static __device__ float ld(bf16_t v) { return bf2f(v); }
    static __device__ bf16_t fin(float acc, float div) {
        bf16_t s = f2bf(acc);
        return div != 0.0f ? f2bf(bf2f(s) / bf2f(f2bf(div))) : s;
    }
};
template <> struct IO<f16_t> {
    static constexpr bool is_bf16 = true;      // "16-bit": f16::from_f32(f32::MIN) is -inf as well (reduction.rs:602,615)
    static __device__ float ld(f16_t v) { return h2f(v); }
    static __device__ f16_t fin(float acc, float div) {
        f16_t s = f2h(acc);
        return div != 0.0f ? f2h(h2f(s) / h2f(f2h(div))) : s;
    }
};

// ---- wave64 butterfly on DPP ------------------------------------------------------------------
template <class R, int CTRL>
__device__ inline float dpp_combine(float v) {
    int iv = __builtin_bit_cast(int, v);
    int ov = __builtin_amdgcn_update_dpp(iv, iv, CTRL, 0xF, 0xF, false);
    return R::op(v, __builtin_bit_cast(float, ov));
}
// After this every lane of a 16-lane row holds the row's result; the four rows are then
// combined in a fixed order through readlane.
template <class R>
__device__ inline float wave_reduce(float v) {
    v = dpp_combine<R, 0xB1>(v);    // quad_perm [1,0,3,2]
    v = dpp_combine<R, 0x4E>(v);    // quad_perm [2,3,0,1]
    v = dpp_combine<R, 0x141>(v);   // row_half_mirror
    v = dpp_combine<R, 0x140>(v);   // row_mirror
    int iv = __builtin_bit_cast(int, v);
    float r0 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 0));
    float r1 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 16));
    float r2 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 32));
    float r3 = __builtin_bit_cast(float, __builtin_amdgcn_readlane(iv, 48));
    return R::op(R::op(r0, r1), R::op(r2, r3));
}

// The same butterfly inside each 16-lane row of the wave (four rows, four results).
template <class R>
__device__ inline float row16_reduce(float v) {
    v = dpp_combine<R, 0xB1>(v);
    v = dpp_combine<R, 0x4E>(v);
    v = dpp_combine<R, 0x141>(v);
    v = dpp_combine<R, 0x140>(v);
    return v;
}

constexpr int RB = 256;

// ---- row reduce: [rows, L] → [rows, chunks] ---------------------------------------------------
// TPR threads cooperate on one (row, chunk): one, a 16-lane row of a wave, a wave, or the block.  VEC > 1 requires L % VEC == 0, chunk_len % VEC == 0
// and a 16-byte aligned base.
// Block and thread index are arguments (the interpreter of recorded programs passes virtual ones); `part`
// is RB / WAVE floats of LDS owned by this (virtual) block.  Every thread reaches the barrier.
// BATCH > 0: the loads of BATCH steps are in flight together whatever the row length (steps past the end are skipped),
// for callers that run a single work-group and pay every memory latency in full; the adds keep the order.
template <class TIn, class TOut, class R, int TPR, int VEC, bool STREAM = false, int BATCH = 0>
__device__ __forceinline__ void row_reduce_body(const TIn* __restrict__ in, TOut* __restrict__ out, size_t rows, size_t L,
                                                unsigned chunks, size_t chunk_len, float div, bool src_bf16, unsigned bid,
                                                unsigned tid, float* part, float* mirror = nullptr) {
    constexpr int RPB = RB / TPR;
    size_t unit = (size_t)bid * RPB + tid / TPR;   // (row, chunk) pair
    const unsigned t = tid % TPR;
    size_t total = rows * chunks;
    float acc = R::init(src_bf16);
    if (unit < total) {
        size_t row = unit / chunks, chunk = unit % chunks;
        size_t beg = chunk * chunk_len, end = beg + chunk_len < L ? beg + chunk_len : L;
        const TIn* src = in + row * L;
        if constexpr (VEC > 1) {
            float a[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) a[e] = R::init(src_bf16);
            // four loads in flight per lane; the adds keep the order of the plain loop
            constexpr size_t STEP = (size_t)TPR * VEC;
            size_t i = beg + (size_t)t * VEC;
            if constexpr (BATCH > 0) {
                for (; i < end; i += BATCH * STEP) {
                    AVec<TIn, VEC> v[BATCH];
#pragma unroll
                    for (int k = 0; k < BATCH; ++k)      // steps past the end re-read the first (an unconditional load, not added)
                        v[k] = *(const AVec<TIn, VEC>*)(src + (i + k * STEP < end ? i + k * STEP : i));
#pragma unroll
                    for (int k = 0; k < BATCH; ++k)
                        if (i + k * STEP < end)
#pragma unroll
                            for (int e = 0; e < VEC; ++e) a[e] = R::op(a[e], IO<TIn>::ld(v[k].v[e]));
                }
            }
            for (; i + 3 * STEP < end; i += 4 * STEP) {
                AVec<TIn, VEC> v[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) v[k] = ld_vec<STREAM>((const AVec<TIn, VEC>*)(src + i + k * STEP));
#pragma unroll
                for (int k = 0; k < 4; ++k)
#pragma unroll
                    for (int e = 0; e < VEC; ++e) a[e] = R::op(a[e], IO<TIn>::ld(v[k].v[e]));
            }
            for (; i < end; i += STEP) {
                AVec<TIn, VEC> v = *(const AVec<TIn, VEC>*)(src + i);
#pragma unroll
                for (int e = 0; e < VEC; ++e) a[e] = R::op(a[e], IO<TIn>::ld(v.v[e]));
            }
#pragma unroll
            for (int e = 0; e < VEC; ++e) acc = R::op(acc, a[e]);
        } else if constexpr (BATCH > 0) {
            for (size_t i = beg + t; i < end; i += (size_t)BATCH * TPR) {
                TIn v[BATCH];
#pragma unroll
                for (int k = 0; k < BATCH; ++k) v[k] = src[i + (size_t)k * TPR < end ? i + (size_t)k * TPR : i];
#pragma unroll
                for (int k = 0; k < BATCH; ++k)
                    if (i + (size_t)k * TPR < end) acc = R::op(acc, IO<TIn>::ld(v[k]));
            }
        } else {
            for (size_t i = beg + t; i < end; i += TPR) acc = R::op(acc, IO<TIn>::ld(src[i]));
        }
    }
    if constexpr (TPR >= WAVE) acc = wave_reduce<R>(acc);
    else if constexpr (TPR == 16) acc = row16_reduce<R>(acc);
    if constexpr (TPR > WAVE) {
        if (tid % WAVE == 0) part[tid / WAVE] = acc;
        __syncthreads();
        acc = part[0];
#pragma unroll
        for (int w = 1; w < RB / WAVE; ++w) acc = R::op(acc, part[w]);
    }
    if (t == 0 && unit < total) {
        const TOut res = IO<TOut>::fin(acc, div);
        out[unit] = res;
        if constexpr (std::is_same<TOut, float>::value)
            if (mirror) mirror[unit] = res;      // LDS copy of the results for the caller's later stages
    }
}
template <class TIn, class TOut, class R, int TPR, int VEC, bool STREAM = false>
__global__ __launch_bounds__(RB) void row_reduce_kernel(const TIn* __restrict__ in, TOut* __restrict__ out, size_t rows,
                                                        size_t L, unsigned chunks, size_t chunk_len, float div,
                                                        bool src_bf16) {
    __shared__ float part[RB / WAVE];
    row_reduce_body<TIn, TOut, R, TPR, VEC, STREAM>(in, out, rows, L, chunks, chunk_len, div, src_bf16, blockIdx.x, threadIdx.x, part);
}
// Argument block of one recorded row_reduce launch; instantiation number of (reducer, threads per row, vector form).
struct RowProgArgs {
    const void* in;
    void* out;
    size_t rows, L;
    unsigned chunks;
    size_t chunk_len;
    float div;
    bool src_bf16;
};
template <class R> struct ReducerIndex;
template <> struct ReducerIndex<RSum> { static constexpr int value = 0; };
template <> struct ReducerIndex<RMax> { static constexpr int value = 1; };
template <> struct ReducerIndex<RMin> { static constexpr int value = 2; };
template <int TPR> struct TprIndex;
template <> struct TprIndex<1> { static constexpr int value = 0; };
template <> struct TprIndex<WAVE> { static constexpr int value = 1; };
template <> struct TprIndex<RB> { static constexpr int value = 2; };
template <class R, int TPR> constexpr uint32_t row_prog_sub(int vec) { return (uint32_t)((ReducerIndex<R>::value * 3 + TprIndex<TPR>::value) * 2 + vec); }

}  // namespace mxh
