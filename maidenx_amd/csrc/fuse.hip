// The kernel behind a fused chain of small launches: in the parallel phase every thread owns one vector (or element) of
// the shared index space and applies the members to it in order; the work-group that finishes last runs the tail.
#include <cstring>
#include <utility>

#include "elementwise.hpp"
#include "fuse.hpp"
#include "fuse_ops.hpp"
#include "gemm_small.hpp"
#include "loss.hpp"
#include "mxh.hpp"
#include "ops.hpp"
#include "reduce_row.hpp"

namespace mxh {

// Operand pointers come out of the chain description, where the compiler cannot know that they point to device memory;
// told so, it uses global loads and stores, which (unlike the generic kind) do not make every later wait for an LDS
// read also wait for the memory access.
typedef __attribute__((address_space(1))) float GFloat;
typedef __attribute__((address_space(1))) const float GCFloat;
typedef float F4 __attribute__((ext_vector_type(4)));
template <int VEC>
__device__ __forceinline__ AVec<float, VEC> gload(GCFloat* p) {
    AVec<float, VEC> r;
    if constexpr (VEC == 4) {
        const F4 t = *(__attribute__((address_space(1))) const F4*)p;
        r.v[0] = t.x; r.v[1] = t.y; r.v[2] = t.z; r.v[3] = t.w;
    } else {
        static_assert(VEC == 1, "16-byte vectors or single elements");
        r.v[0] = p[0];
    }
    return r;
}
template <int VEC>
__device__ __forceinline__ void gstore(GFloat* p, const AVec<float, VEC>& v) {
    if constexpr (VEC == 4) {
        F4 t;
        t.x = v.v[0]; t.y = v.v[1]; t.z = v.v[2]; t.w = v.v[3];
        *(__attribute__((address_space(1))) F4*)p = t;
    } else {
        p[0] = v.v[0];
    }
}
__device__ __forceinline__ GCFloat* gl(const void* p) { return (GCFloat*)(uintptr_t)p; }
__device__ __forceinline__ GFloat* gl(void* p) { return (GFloat*)(uintptr_t)p; }

// the fields of a FuseGroup ahead of its members
struct FuseHead {
    uint32_t n, ndims, vec, ntail;
    uint32_t dims[2];
    FastDiv div_inner;
    size_t nvec;
    uint32_t* ticket;
    uint32_t prefetch, blocks, pad[2];
};
static_assert(sizeof(FuseHead) <= offsetof(FuseGroup, cmd) && offsetof(FuseHead, ticket) == offsetof(FuseGroup, ticket) &&
              offsetof(FuseHead, blocks) == offsetof(FuseGroup, blocks), "FuseHead mirrors FuseGroup");
// the fields of a TailCmd ahead of its argument block
struct TailHead {
    uint32_t kind, sub, sync, fwd;
    int32_t moff0, moff1;
    uint32_t mirrored, pad;
};
static_assert(sizeof(TailHead) == offsetof(TailCmd, arg) && offsetof(TailCmd, moff) == offsetof(TailHead, moff0), "TailHead mirrors TailCmd");
// A barrier that orders the work-group's LDS traffic and nothing else: __syncthreads() also waits for every global
// store the wave has in flight, which a stage that only meets LDS data has no reason to do.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// element offset of thread `v`'s element of a tail stage's own space, for the operand with strides s
// (fields are named one by one, never indexed by a run-time value: the command then stays in scalar registers)
__device__ __forceinline__ int64_t tail_elem(const FuseCmd& c, int64_t s0, int64_t s1, uint32_t v) {
    if (c.ndims == 2) {
        const uint32_t c0 = v / c.dims[1], c1 = v - c0 * c.dims[1];
        return (int64_t)c0 * s0 + (int64_t)c1 * s1;
    }
    return (int64_t)v * s0;
}

// ---- the serial phase: stages run by one work-group ----------------------------------------------------------
// Data between stages travels through LDS: a stage's outputs (at most 256) are mirrored in `mir`, inputs that nothing in
// the tail writes are fetched from memory all at once when the tail starts (`pre`), so that a stage costs LDS latencies
// and not a round trip to memory.  Every output is still stored to memory, without anybody waiting for the store.
constexpr int TAIL_SLOT = 256;
static_assert(MSE_THREADS == EW_BLOCK, "the fused MSE sum is a stage of the tail with its own work-group's thread count");
template <int TPR>
__device__ __forceinline__ void tail_row(uint32_t vec, const RowProgArgs& a, unsigned tid, float* part, float* mirror) {
    if (vec) row_reduce_body<float, float, RSum, TPR, 4, false, 16>((const float*)a.in, (float*)a.out, a.rows, a.L, a.chunks, a.chunk_len, a.div, a.src_bf16, 0, tid, part, mirror);
    else row_reduce_body<float, float, RSum, TPR, 1, false, 16>((const float*)a.in, (float*)a.out, a.rows, a.L, a.chunks, a.chunk_len, a.div, a.src_bf16, 0, tid, part, mirror);
}

__device__ __forceinline__ void run_tail(const FuseGroup& sg, uint32_t ntail, uint32_t want, unsigned tid, float* part, float* mir, float* pre) {
    // `want`: which (stage, input) pairs are fetched up front
    if (want) {
        float got[2 * FUSE_MAX_TAIL];
#pragma unroll
        for (int k = 0; k < FUSE_MAX_TAIL; ++k) {
            got[2 * k] = got[2 * k + 1] = 0.0f;
            if ((want >> (2 * k)) & 3u) {
                const FuseCmd c = lds_uniform<FuseCmd>(sg.tail[k].arg);
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    if (((want >> (2 * k + j)) & 1u) && tid < c.nel) got[2 * k + j] = gl(c.in[j])[tail_elem(c, c.is[j][0], c.is[j][1], tid)];
            }
        }
#pragma unroll
        for (int q = 0; q < 2 * FUSE_MAX_TAIL; ++q)
            if (want & (1u << q)) pre[q * TAIL_SLOT + tid] = got[q];
    }
    float prev = 0.0f;            // what this thread wrote in the stage before (an elementwise stage of the same layout)
    for (uint32_t k = 0; k < ntail; ++k) {
        const TailHead t = lds_uniform<TailHead>(&sg.tail[k]);
        if (t.sync == 2) __syncthreads();
        else if (t.sync == 1) lds_barrier();
        float* mirror = t.mirrored ? mir + k * TAIL_SLOT : nullptr;
        if (t.kind == TAIL_EW) {
            const FuseCmd c = lds_uniform<FuseCmd>(sg.tail[k].arg);
            if (tid < c.nel) {
                float val[2][1] = {{0.0f}, {0.0f}};
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    if (j >= (int)c.nin) continue;
                    if (t.fwd & (1u << j)) { val[j][0] = prev; continue; }
                    const uint32_t from = (c.src >> (8 * j)) & 0xFFu;
                    const int64_t at = tail_elem(c, c.is[j][0], c.is[j][1], tid);
                    if (from == FUSE_SRC_MEMORY) val[j][0] = pre[(2 * k + j) * TAIL_SLOT + tid];
                    else if (from == FUSE_SRC_MEMORY_LATE) val[j][0] = gl(c.in[j])[at];
                    else val[j][0] = mir[from * TAIL_SLOT + (j ? t.moff1 : t.moff0) + at];
                }
                float r[1] = {0.0f};
                fuse_apply<1>(c.op, val[0], val[1], r, c.payload);
                gl(c.out)[tail_elem(c, c.os[0], c.os[1], tid)] = r[0];
                if (mirror) mirror[tid] = r[0];
                prev = r[0];
            }
        } else if (t.kind == TAIL_ROW_REDUCE) {
            const RowProgArgs a = lds_uniform<RowProgArgs>(sg.tail[k].arg);
            const uint32_t vec = t.sub & 1u, tpr = (t.sub >> 1) % 3;        // the reducer is RSum: nothing else is recorded
            if (tpr == 0) tail_row<1>(vec, a, tid, part, mirror);
            else if (tpr == 1) tail_row<WAVE>(vec, a, tid, part, mirror);
            else tail_row<RB>(vec, a, tid, part, mirror);
        } else if (t.kind == TAIL_MSE) {
            const MseArgs a = lds_uniform<MseArgs>(sg.tail[k].arg);
            const float sum = mse_block_sum(a.pred, a.target, (size_t)a.n, 0, 1, tid, part);
            if (tid == 0) {
                const float loss = OpDivScalar<float>{(float)(size_t)a.n}(sum);
                gl((void*)a.loss)[0] = loss;
                if (mirror) mirror[0] = loss;
            }
        } else {
            const GemmArgs g = lds_uniform<GemmArgs>(sg.tail[k].arg);
            const unsigned outputs = g.I * g.J * g.batch;
            if (t.sub == 2) {            // one wave per output, the waves of the group taking the outputs in turn
                for (unsigned o = tid / WAVE; o < outputs; o += EW_BLOCK / WAVE) gemm_wavedot_body<float>(g, o, (int)(tid % WAVE), mirror);
            } else if (t.sub == 1) gemm_rowsdot_any<EW_BLOCK>(g, tid, part, mirror);        // the eager path's choice, made on the host
            else for (unsigned o = 0; o < outputs; o += 4) {
                if (o) __syncthreads();              // the fold of the outputs before still reads `part`
                gemm_blockdot_body<float, EW_BLOCK, 4>(g, o, outputs, tid, part, mirror);
            }
        }
    }
}

// ---- the chain kernel ----------------------------------------------------------------------------------------
template <int VEC>
__global__ __launch_bounds__(EW_BLOCK) void ew_group_kernel(FuseGroup g) {
    // The chain description is 3.5 KB of kernel arguments; read member by member it costs a scalar-cache miss per
    // member.  Copy it to LDS once (every thread one 16-byte piece: one memory latency) and walk it there.
    __shared__ FuseGroup sg;
    __shared__ float part[4 * EW_BLOCK / WAVE];      // four outputs of a tail matmul side by side
    __shared__ uint32_t last_group;
    // Outputs of the parallel phase wait here, one slot per member and thread, until all members are done: on this
    // hardware a wave that waits for a load also waits for every store it issued before, so a member that stored
    // right away would make the next one that loads sit out the store's round trip.  The tail reuses the space.
    constexpr int STAGE = FUSE_MAX_CMDS * EW_BLOCK * (VEC + 2);      // values and the addresses they go to
    constexpr int POOL = STAGE > 3 * FUSE_MAX_TAIL * TAIL_SLOT ? STAGE : 3 * FUSE_MAX_TAIL * TAIL_SLOT;
    __shared__ __attribute__((aligned(16))) float pool[POOL];
    {
        typedef uint32_t Piece __attribute__((ext_vector_type(4)));
        typedef const __attribute__((address_space(4))) Piece* ArgPtr;
        ArgPtr src = (ArgPtr)__builtin_amdgcn_kernarg_segment_ptr();
        static_assert(sizeof(FuseGroup) % 16 == 0 && sizeof(FuseGroup) <= 16 * EW_BLOCK, "one 16-byte piece per thread");
        if (threadIdx.x < sizeof(FuseGroup) / 16) ((Piece*)&sg)[threadIdx.x] = src[threadIdx.x];
    }
    __syncthreads();
    // From here on everything comes from the LDS copy: a kernel argument read where it is first needed is a scalar load
    // that misses its cache, a microsecond each time.
    const FuseHead h = lds_uniform<FuseHead>(&sg);
    const size_t v = (size_t)blockIdx.x * EW_BLOCK + threadIdx.x;
    if (v < h.nvec) {
        // coordinates of this thread's first element over (outer, inner); one dim: everything is "inner"
        uint32_t c0 = 0, c1 = (uint32_t)v * VEC;
        const uint32_t ndims = h.ndims;
        if (ndims == 2) fd_divmod((uint32_t)v * VEC, h.div_inner, c0, c1);
        AVec<float, VEC>* staged = (AVec<float, VEC>*)pool + threadIdx.x;      // + member * EW_BLOCK
        float** where = (float**)(pool + FUSE_MAX_CMDS * EW_BLOCK * VEC) + threadIdx.x;      // where each staged output goes
        AVec<float, VEC> r;          // what the previous member wrote at this thread's elements
#pragma unroll
        for (int e = 0; e < VEC; ++e) r.v[e] = 0.0f;
        for (uint32_t k = 0; k < h.n; ++k) {
            const FuseCmd c = lds_uniform<FuseCmd>(&sg.cmd[k]);
            if (c.op == FUSE_OP_DOT) {
                // one output per element, r ascending, multiply and add unfused: gemm_thread_body's order
                const uint32_t J = c.dims[0], R = c.dims[1];
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const uint32_t idx = (uint32_t)v * VEC + e;
                    const uint32_t i = idx / J, j = idx - i * J;
                    GCFloat* x = gl(c.in[0]) + (int64_t)i * c.is[0][0];
                    GCFloat* y = gl(c.in[1]) + (int64_t)j * c.is[1][1];
                    float acc = 0.0f;
                    for (uint32_t q = 0; q < R; ++q) acc = acc + x[(int64_t)q * c.is[0][1]] * y[(int64_t)q * c.is[1][0]];
                    r.v[e] = acc;
                }
            } else {
                float val[2][VEC];
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    if (j >= (int)c.nin) {
#pragma unroll
                        for (int e = 0; e < VEC; ++e) val[j][e] = 0.0f;
                        continue;
                    }
                    if (c.fwd & (1u << j)) {         // the value is still in registers
#pragma unroll
                        for (int e = 0; e < VEC; ++e) val[j][e] = r.v[e];
                        continue;
                    }
                    const uint32_t from = (c.src >> (8 * j)) & 0xFFu;
                    if (from != FUSE_SRC_MEMORY) {   // an earlier member's output, element for element: still staged
                        const AVec<float, VEC> t = staged[from * EW_BLOCK];
#pragma unroll
                        for (int e = 0; e < VEC; ++e) val[j][e] = t.v[e];
                        continue;
                    }
                    const int64_t s = ndims == 2 ? c.is[j][1] : c.is[j][0];
                    GCFloat* src = gl(c.in[j]) + (ndims == 2 ? (int64_t)c0 * c.is[j][0] : 0) + (int64_t)c1 * s;
                    if (VEC > 1 && s == 1) {
                        const AVec<float, VEC> t = gload<VEC>(src);
#pragma unroll
                        for (int e = 0; e < VEC; ++e) val[j][e] = t.v[e];
                    } else if (s == 0) {
                        const float t = src[0];
#pragma unroll
                        for (int e = 0; e < VEC; ++e) val[j][e] = t;
                    } else {
#pragma unroll
                        for (int e = 0; e < VEC; ++e) val[j][e] = src[(int64_t)e * s];
                    }
                }
                if (c.op == FUSE_OP_MSE_BACKWARD) {
                    const uint64_t seed = ((uint64_t)c.payload[1] << 32) | c.payload[0];      // (0: the gradient of the loss is 1)
                    const float scale = mse_grad_scale(seed ? gl((const void*)seed)[0] : 1.0f, (float)c.nel);
#pragma unroll
                    for (int e = 0; e < VEC; ++e) r.v[e] = mse_grad(scale, val[0][e], val[1][e]);
                } else {
                    fuse_apply<VEC>(c.op, val[0], val[1], r.v, c.payload);
                }
            }
            staged[k * EW_BLOCK] = r;
            where[k * EW_BLOCK] = (float*)c.out + (ndims == 2 ? (int64_t)c0 * c.os[0] + (int64_t)c1 * c.os[1] : (int64_t)c1 * c.os[0]);
        }
        // every member's output to memory, in member order (a later member may write where an earlier one did)
        for (uint32_t k0 = 0; k0 < h.n; k0 += 4) {
            AVec<float, VEC> o[4];
            float* dst[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t k = k0 + i < h.n ? k0 + i : k0;
                o[i] = staged[k * EW_BLOCK];
                dst[i] = where[k * EW_BLOCK];
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (k0 + i < h.n) {
                    gstore<VEC>(gl(dst[i]), o[i]);
                }
            }
        }
    }
    if (h.ntail == 0) return;
    if (h.blocks > 1) {
        // Publish this work-group's writes to the whole device, then draw a ticket.  The group that draws the last one
        // knows every other group has published; it alone goes on.  Nobody waits for anybody.
        __threadfence();
        __syncthreads();
        if (threadIdx.x == 0) {
            const uint32_t drawn = atomicAdd(h.ticket, 1u);
            last_group = drawn == h.blocks - 1 ? 1u : 0u;
        }
        __syncthreads();
        if (!last_group) return;
        __threadfence();
    } else {
        __syncthreads();          // the tail reads what other threads of this group stored, and reuses the staging space
    }
    run_tail(sg, h.ntail, h.prefetch, threadIdx.x, part, pool, pool + FUSE_MAX_TAIL * TAIL_SLOT);
    if (h.blocks > 1 && threadIdx.x == 0) atomicExch(h.ticket, 0u);      // for the next launch of this or any other chain
}

// The tickets live in the code object: nothing to allocate or free, zero when the module is loaded, and every chain
// leaves its slot at zero again.
static __device__ uint32_t g_ticket_slots[FUSE_TICKETS];
uint32_t* fuse_tickets() {
    uint32_t* p = nullptr;
    if (hipGetSymbolAddress((void**)&p, HIP_SYMBOL(g_ticket_slots)) != hipSuccess) {
        (void)hipGetLastError();
        return nullptr;
    }
    return p;
}

void fuse_launch(const FuseGroup& g, void* stream_) {
    const unsigned blocks = g.n ? cdiv(g.nvec, (size_t)EW_BLOCK) : 1u;
    FuseGroup launch = g;
    launch.blocks = blocks;
    if (g.vec) hipLaunchKernelGGL(ew_group_kernel<4>, dim3(blocks), dim3(EW_BLOCK), 0, (hipStream_t)stream_, launch);
    else hipLaunchKernelGGL(ew_group_kernel<1>, dim3(blocks), dim3(EW_BLOCK), 0, (hipStream_t)stream_, launch);
    MXH_HIP(hipGetLastError());
}

}  // namespace mxh
