// Operand description of a matmul, the element codecs and the two kernels for very small products: shared by
// the GEMM dispatch and by the interpreter of recorded programs.
#pragma once
#include "mxh.hpp"
#include "reduce_row.hpp"

namespace mxh {

struct GemmArgs {
    const void* X;
    const void* Y;
    void* out;
    int64_t xb, xi, xr;   // element strides of X: batch, output row, reduction
    int64_t yb, yr, yj;   // element strides of Y: batch, reduction, output column
    uint32_t I, J, R, batch;
    uint32_t tiles_i, tiles_j;
    // split-K: the reduction is cut into `splits` chunks of r_chunk (a multiple of the k-tile); with splits > 1
    // every block writes its f32 partial tile to part[split][batch*I*J] and a second kernel folds them
    uint32_t splits, r_chunk;
    float* part;
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
template <> struct Elem<f16_t> {
    static constexpr int VEC = 8;
    static __device__ float ld(f16_t v) { return h2f(v); }
    static __device__ f16_t st(float v) { return f2h(v); }
    static __device__ f16_t zero() { return f16_t{0}; }
};

constexpr int GB = 256;          // threads per block of the small-shape kernels

// ---- small shapes -----------------------------------------------------------------------------------
// One thread per output element, r ascending, multiply and add unfused: the reference's own
// order, so f32 results are bit-identical to it.
template <class T>
__device__ __forceinline__ void gemm_thread_body(const GemmArgs& g, unsigned bid, unsigned tid) {
    size_t idx = (size_t)bid * GB + tid;
    size_t per = (size_t)g.I * g.J;
    if (idx >= per * g.batch) return;
    uint32_t b = (uint32_t)(idx / per);
    uint32_t rem = (uint32_t)(idx % per);
    uint32_t i = rem / g.J, j = rem % g.J;
    const T* x = (const T*)g.X + (int64_t)b * g.xb + (int64_t)i * g.xi;
    const T* y = (const T*)g.Y + (int64_t)b * g.yb + (int64_t)j * g.yj;
    float acc = 0.0f;
    // eight terms' operands requested together (one memory latency instead of eight), added in ascending r as before
    constexpr int Q = 8;
    uint32_t r = 0;
    for (; r + Q <= g.R; r += Q) {
        float xv[Q], yv[Q];
#pragma unroll
        for (int k = 0; k < Q; ++k) {
            xv[k] = Elem<T>::ld(x[(int64_t)(r + k) * g.xr]);
            yv[k] = Elem<T>::ld(y[(int64_t)(r + k) * g.yr]);
        }
#pragma unroll
        for (int k = 0; k < Q; ++k) acc = acc + xv[k] * yv[k];
    }
    for (; r < g.R; ++r) acc = acc + Elem<T>::ld(x[(int64_t)r * g.xr]) * Elem<T>::ld(y[(int64_t)r * g.yr]);
    ((T*)g.out)[idx] = Elem<T>::st(acc);
}
template <class T>
__global__ __launch_bounds__(GB) void gemm_thread_kernel(GemmArgs g) { gemm_thread_body<T>(g, blockIdx.x, threadIdx.x); }

// One wave per output element `idx`: lanes stride over r, 4 independent partial sums per lane, then a fixed shuffle tree.
// Every lane of the wave calls it; `mirror` (may be null): LDS copy of the outputs, element idx.
template <class T>
__device__ __forceinline__ void gemm_wavedot_body(const GemmArgs& g, size_t idx, int lane, float* mirror) {
    size_t per = (size_t)g.I * g.J;
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
    if (live && lane == 0) {
        ((T*)g.out)[idx] = Elem<T>::st(acc);
        if (mirror) mirror[idx] = acc;
    }
}

// The same sums for Y with unit column stride and J a multiple of the 16-byte vector: a thread owns VEC neighbouring
// outputs of one row (one vector load of Y per term, one vector store), blockIdx.y is the batch, and nothing is divided
// in 64 bits - with a short reduction the kernel above spends its time on its index arithmetic ([4096,8] x [8,4096]:
// 90 us for 64 MB of output).  Every output is still its terms in ascending r, multiply and add unfused.
template <class T>
__global__ __launch_bounds__(GB) void gemm_thread_vec_kernel(GemmArgs g) {
    constexpr int VEC = 16 / sizeof(T);
    const uint32_t jv = g.J / VEC;                        // vectors per output row
    const uint32_t v = blockIdx.x * GB + threadIdx.x;
    if (v >= g.I * jv) return;
    const uint32_t i = v / jv, j = (v % jv) * VEC, b = blockIdx.y;
    const T* x = (const T*)g.X + (int64_t)b * g.xb + (int64_t)i * g.xi;
    const T* y = (const T*)g.Y + (int64_t)b * g.yb + j;
    float acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] = 0.0f;
    for (uint32_t r = 0; r < g.R; ++r) {
        const float a = Elem<T>::ld(x[(int64_t)r * g.xr]);
        const AVec<T, VEC> yv = *(const AVec<T, VEC>*)(y + (int64_t)r * g.yr);
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] = acc[e] + a * Elem<T>::ld(yv.v[e]);
    }
    AVec<T, VEC> o;
#pragma unroll
    for (int e = 0; e < VEC; ++e) o.v[e] = Elem<T>::st(acc[e]);
    *(AVec<T, VEC>*)((T*)g.out + ((size_t)b * g.I + i) * g.J + j) = o;
}
// whether the vector form applies
template <class T>
inline bool gemm_thread_vec_ok(const GemmArgs& g) {
    constexpr int VEC = 16 / sizeof(T);
    return g.yj == 1 && g.J % VEC == 0 && g.yr % VEC == 0 && g.yb % VEC == 0 && (uintptr_t)g.Y % 16 == 0 && (uintptr_t)g.out % 16 == 0 &&
           g.batch <= 65535 && (size_t)g.I * (g.J / VEC) < (1ull << 32) && (size_t)g.I * g.J >= 65536;
}

// One block per output element for a handful of outputs with a long reduction (the MLP's weight gradient:
// 3 outputs of 10000 terms): NT threads stride over r, waves fold by a DPP butterfly, the block by LDS, in a fixed order.
// `part`: NT / WAVE floats of LDS per output reduced side by side; every thread of the block reaches the barrier (threads at and beyond NT, which a
// larger work-group may have, contribute nothing).  NT is a function of the reduction length alone, so that every path
// that runs this body for a given product - the kernel below, a recorded program, the tail of a fused chain - adds in
// the same order.
constexpr uint32_t BLOCKDOT_WIDE_R = 32768;      // reductions from this length on use 1024 threads, shorter ones 256
inline unsigned blockdot_threads(uint32_t R) { return R >= BLOCKDOT_WIDE_R ? 1024u : 256u; }
// NO outputs (bid .. bid + NO - 1, those below `outputs`) are reduced side by side, and the loads of 8 terms of each
// are in flight together: the terms of an output are still added in ascending r per thread.
template <class T, int NT, int NO = 1>
__device__ __forceinline__ void gemm_blockdot_body(const GemmArgs& g, unsigned bid, unsigned outputs, unsigned tid, float* part, float* mirror = nullptr) {
    constexpr int U = 8;
    const size_t per = (size_t)g.I * g.J;
    const uint32_t R = g.R;
    const int64_t xstep = (int64_t)NT * g.xr, ystep = (int64_t)NT * g.yr;      // pointers advance by additions only
    const T* x[NO];
    const T* y[NO];
    float acc[NO];
    bool live[NO];
#pragma unroll
    for (int o = 0; o < NO; ++o) {
        live[o] = bid + o < outputs;
        const size_t idx = live[o] ? bid + o : bid;
        const uint32_t b = (uint32_t)(idx / per), rem = (uint32_t)(idx % per);
        const uint32_t i = rem / g.J, j = rem % g.J;
        x[o] = (const T*)g.X + (int64_t)b * g.xb + (int64_t)i * g.xi + (int64_t)tid * g.xr;
        y[o] = (const T*)g.Y + (int64_t)b * g.yb + (int64_t)j * g.yj + (int64_t)tid * g.yr;
        acc[o] = 0.0f;
    }
    if (tid < (unsigned)NT) {
        for (uint32_t r0 = tid; r0 < R; r0 += U * NT) {
            float p[NO][U];
#pragma unroll
            for (int o = 0; o < NO; ++o) {
                if (!live[o]) continue;                      // uniform over the work-group
                const T* xp = x[o];
                const T* yp = y[o];
#pragma unroll
                for (int k = 0; k < U; ++k) {
                    // steps past the end re-read the step before (an unconditional load; its product is not added)
                    p[o][k] = Elem<T>::ld(*xp) * Elem<T>::ld(*yp);
                    if (r0 + (k + 1) * NT < R) { xp += xstep; yp += ystep; }
                }
                x[o] += U * xstep;
                y[o] += U * ystep;
            }
#pragma unroll
            for (int o = 0; o < NO; ++o) {
                if (!live[o]) continue;
#pragma unroll
                for (int k = 0; k < U; ++k)
                    if (r0 + k * NT < R) acc[o] += p[o][k];
            }
        }
#pragma unroll
        for (int o = 0; o < NO; ++o) {
            acc[o] = wave_reduce<RSum>(acc[o]);      // the butterfly on DPP: a dozen instructions, no trips through LDS
            if (tid % WAVE == 0) part[o * (NT / WAVE) + tid / WAVE] = acc[o];
        }
    }
    __syncthreads();
    if (tid < (unsigned)NO && bid + tid < outputs) {
        float sum = 0.0f;
#pragma unroll
        for (int w = 0; w < NT / WAVE; ++w) sum += part[tid * (NT / WAVE) + w];
        ((T*)g.out)[bid + tid] = Elem<T>::st(sum);
        if (mirror) mirror[bid + tid] = sum;      // LDS copy of the results for the caller's later stages
    }
}
// out[j] = sum over r of X[r] * Y[r, j] for a contiguous f32 X and a row-major Y of J <= 4 columns: the weight gradient of a
// layer with one output feature ([1,R] x [R,J]).  One block does all J outputs.  Thread t owns rows 4t .. 4t+3 of every
// 4 * NT rows, so one 16-byte load brings four terms of X and J of them the 4 * J matching terms of Y (the strided form
// above needs 4 + 4 * J scalar loads for the same terms); the loads of ten such groups are in flight together.  A thread
// adds the terms of an output in ascending r; waves fold by a DPP butterfly, the block by LDS, in a fixed order.
// `part`: J * NT / WAVE floats of LDS.
// The same with the operands' roles exchanged ([J,R] x [R,1] with a column-major left operand: what matmul_backward asks
// for as A^T . dC) is the same sum, a product of two floats not depending on their order: rowsdot_normalise() turns it
// into the first form.
__host__ __device__ inline bool rowsdot_normalise(GemmArgs& g) {
    if (g.batch != 1 || g.R % 4 != 0 || g.R < 4096 || g.R >= BLOCKDOT_WIDE_R) return false;
    if (g.J == 1 && g.I >= 1 && g.I <= 4 && g.xi == 1 && g.xr == (int64_t)g.I && g.yr == 1) {
        // out[i] = sum_r X[r, i] * Y[r]: X is the row-major matrix, Y the vector
        const void* m = g.X;
        g.X = g.Y;
        g.Y = m;
        g.J = g.I;
        g.I = 1;
        g.xr = 1;
        g.yr = (int64_t)g.J;
        g.yj = 1;
    }
    return g.I == 1 && g.J >= 1 && g.J <= 4 && g.yj == 1 && g.yr == (int64_t)g.J && g.xr == 1 && ((uintptr_t)g.X % 16) == 0 &&
           ((uintptr_t)g.Y % 16) == 0;
}
inline bool rowsdot_applies(const GemmArgs& g) {
    GemmArgs n = g;
    return rowsdot_normalise(n);
}
// G: groups whose loads are in flight together (it does not change the order of the additions).
template <int NT, int J, int G = 10>
__device__ __forceinline__ void gemm_rowsdot_body(const GemmArgs& g, unsigned tid, float* part, float* mirror = nullptr) {
    // G = 10: 10 * (1 + J) 16-byte loads in flight per thread, a 10240-row product in one round trip
    typedef float F4 __attribute__((ext_vector_type(4)));
    const F4* X4 = (const F4*)g.X;
    const F4* Y4 = (const F4*)g.Y;
    const uint32_t groups = g.R / 4;
    float acc[J];
#pragma unroll
    for (int j = 0; j < J; ++j) acc[j] = 0.0f;
    if (tid < (unsigned)NT) {
        for (uint32_t q0 = tid; q0 < groups; q0 += G * NT) {
            F4 xv[G];
            F4 yv[G][J];
#pragma unroll
            for (int i = 0; i < G; ++i) {
                const uint32_t q = q0 + i * NT < groups ? q0 + i * NT : q0;      // past the end: re-read the first (not added)
                xv[i] = X4[q];
#pragma unroll
                for (int jj = 0; jj < J; ++jj) yv[i][jj] = Y4[(size_t)q * J + jj];
            }
#pragma unroll
            for (int i = 0; i < G; ++i)
                if (q0 + i * NT < groups) {
#pragma unroll
                    for (int rr = 0; rr < 4; ++rr)
#pragma unroll
                        for (int j = 0; j < J; ++j) acc[j] += xv[i][rr] * yv[i][(rr * J + j) / 4][(rr * J + j) % 4];
                }
        }
#pragma unroll
        for (int j = 0; j < J; ++j) {
            acc[j] = wave_reduce<RSum>(acc[j]);
            if (tid % WAVE == 0) part[j * (NT / WAVE) + tid / WAVE] = acc[j];
        }
    }
    __syncthreads();
    if (tid < (unsigned)J) {
        float sum = 0.0f;
#pragma unroll
        for (int w = 0; w < NT / WAVE; ++w) sum += part[tid * (NT / WAVE) + w];
        ((float*)g.out)[tid] = sum;
        if (mirror) mirror[tid] = sum;
    }
}
template <int NT, int G = 10>
__device__ __forceinline__ void gemm_rowsdot_any(const GemmArgs& args, unsigned tid, float* part, float* mirror = nullptr) {
    GemmArgs g = args;
    rowsdot_normalise(g);
    if (g.J == 1) gemm_rowsdot_body<NT, 1, G>(g, tid, part, mirror);
    else if (g.J == 2) gemm_rowsdot_body<NT, 2, G>(g, tid, part, mirror);
    else if (g.J == 3) gemm_rowsdot_body<NT, 3, G>(g, tid, part, mirror);
    else gemm_rowsdot_body<NT, 4, G>(g, tid, part, mirror);
}
template <class T, int NT>
__global__ __launch_bounds__(NT) void gemm_blockdot_kernel(GemmArgs g) {
    __shared__ float part[NT / WAVE];
    gemm_blockdot_body<T, NT>(g, blockIdx.x, gridDim.x, threadIdx.x, part);
}

}  // namespace mxh
