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
    uint32_t prefetch, blocks, nwide, wide_m, wide_nvec, pad[1];
};
static_assert(sizeof(FuseHead) <= offsetof(FuseGroup, cmd) && offsetof(FuseHead, ticket) == offsetof(FuseGroup, ticket) &&
              offsetof(FuseHead, blocks) == offsetof(FuseGroup, blocks) && offsetof(FuseHead, wide_nvec) == offsetof(FuseGroup, wide_nvec),
              "FuseHead mirrors FuseGroup");
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
    // `want`: which (stage, input) pairs are fetched up front; they go to LDS when the first elementwise stage comes up,
    // so that the stages before it can overlap the fetch
    float got[2 * FUSE_MAX_TAIL];
#pragma unroll
    for (int q = 0; q < 2 * FUSE_MAX_TAIL; ++q) got[q] = 0.0f;
    if (want) {
#pragma unroll
        for (int k = 0; k < FUSE_MAX_TAIL; ++k) {
            if ((want >> (2 * k)) & 3u) {
                const FuseCmd c = lds_uniform<FuseCmd>(sg.tail[k].arg);
#pragma unroll
                for (int j = 0; j < 2; ++j)
                    if (((want >> (2 * k + j)) & 1u) && tid < c.nel) got[2 * k + j] = gl(c.in[j])[tail_elem(c, c.is[j][0], c.is[j][1], tid)];
            }
        }
    }
    bool fetched = want == 0;
    float prev = 0.0f;            // what this thread wrote in the stage before (an elementwise stage of the same layout)
    for (uint32_t k = 0; k < ntail; ++k) {
        const TailHead t = lds_uniform<TailHead>(&sg.tail[k]);
        if (t.kind == TAIL_EW && !fetched) {
#pragma unroll
            for (int q = 0; q < 2 * FUSE_MAX_TAIL; ++q)
                if (want & (1u << q)) pre[q * TAIL_SLOT + tid] = got[q];        // (read back by this thread only)
            fetched = true;
        }
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

// ---- the members of the parallel phase --------------------------------------------------------------------------
// (Element offsets are computed in 32 bits: the host only lets operands in whose elements lie within 2^31 of their base.)
// A matmul producer at unit `u` of its flat output space: one output per element, r ascending, multiply and add
// unfused (gemm_thread_body's order).
template <int VEC>
__device__ __forceinline__ void member_dot(const FuseCmd& c, uint32_t u, AVec<float, VEC>& r) {
    const uint32_t J = c.dims[0], R = c.dims[1];
    uint32_t row[VEC], col[VEC];
    row[0] = (u * VEC) / J;
    col[0] = u * VEC - row[0] * J;
#pragma unroll
    for (int e = 1; e < VEC; ++e) {
        col[e] = col[e - 1] + 1;
        row[e] = row[e - 1];
        if (col[e] == J) { col[e] = 0; ++row[e]; }
    }
    // (term by term: requesting several terms of an element together costs more instructions than it saves latencies
    // for the reductions of one to three terms this is for)
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
        GCFloat* x = gl(c.in[0]) + row[e] * (uint32_t)c.is[0][0];
        GCFloat* y = gl(c.in[1]) + col[e] * (uint32_t)c.is[1][1];
        float acc = 0.0f;
        for (uint32_t q = 0; q < R; ++q) acc = acc + x[q * (uint32_t)c.is[0][1]] * y[q * (uint32_t)c.is[1][0]];
        r.v[e] = acc;
    }
}
// The one-term product of the wide space whose left operand is a first-space member's output, row for row: round q of
// this thread's m = J units.  Its VEC * J outputs are the thread's own VEC rows (`own`, that member's staged output) times
// the J entries of the right operand, so which row and which entry meet at element e of the round is the same for every
// thread.
template <int VEC>
__device__ __forceinline__ void member_dot_own(const FuseCmd& c, uint32_t q, const AVec<float, VEC>& own, AVec<float, VEC>& r) {
    const uint32_t J = c.dims[0];
    const uint32_t yj = (uint32_t)c.is[1][1];
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
        const uint32_t at = q * VEC + e, row = at / J, col = at - row * J;      // (uniform)
        float x = own.v[0];
#pragma unroll
        for (int i = 1; i < VEC; ++i) x = row == (uint32_t)i ? own.v[i] : x;
        r.v[e] = 0.0f + x * gl(c.in[1])[col * yj];
    }
}
// An elementwise member (FUSE_OP_MSE_BACKWARD included) at the VEC elements that start at coordinates (c0, c1).  `r`
// comes in as what the member before wrote at these elements and goes out as this member's values; an input that is
// an earlier member's output is read from that member's staging slot, number `member * slot_mul + slot_add`.
template <int VEC>
__device__ __forceinline__ void member_ew(const FuseCmd& c, uint32_t ndims, uint32_t c0, uint32_t c1, const AVec<float, VEC>* staged,
                                          uint32_t slot_mul, int slot_add, AVec<float, VEC>& r) {
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
            const AVec<float, VEC> t = staged[(uint32_t)((int)(from * slot_mul) + slot_add) * EW_BLOCK];
#pragma unroll
            for (int e = 0; e < VEC; ++e) val[j][e] = t.v[e];
            continue;
        }
        const uint32_t s = (uint32_t)(ndims == 2 ? c.is[j][1] : c.is[j][0]);
        GCFloat* src = gl(c.in[j]) + ((ndims == 2 ? c0 * (uint32_t)c.is[j][0] : 0u) + c1 * s);
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
            for (int e = 0; e < VEC; ++e) val[j][e] = src[(uint32_t)e * s];
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
    AVec<float, VEC>* staged = (AVec<float, VEC>*)pool + threadIdx.x;      // + slot * EW_BLOCK
    float** where = (float**)(pool + FUSE_MAX_CMDS * EW_BLOCK * VEC) + threadIdx.x;      // where each staged output goes
    // One loop over the members of the first space, then over the rounds of the wide space (round-major: a member
    // then finds what the member before it wrote, same round, in registers) - one copy of the member code, so that
    // what the first rounds bring into the instruction cache serves the later ones.  The thread that owns unit v of the
    // first space owns units m v .. m v + m - 1 of the wide one, one per round.
    const uint32_t m = h.wide_m, items = h.n + h.nwide * m;
    const uint32_t slots = items;
    AVec<float, VEC> r;          // what the previous member wrote at this thread's elements
#pragma unroll
    for (int e = 0; e < VEC; ++e) r.v[e] = 0.0f;
    uint32_t c0 = 0, c1 = (uint32_t)v * VEC;      // first space: coordinates over (outer, inner); one dim: everything is "inner"
    if (h.ndims == 2) fd_divmod((uint32_t)v * VEC, h.div_inner, c0, c1);
    const bool in_space = v < h.nvec;
    uint32_t k = 0, q = 0;
    for (uint32_t it = 0; it < items; ++it) {
        const bool first = it < h.n;
        if (it == h.n) k = h.n;
        const uint32_t unit = first ? (uint32_t)v : (uint32_t)v * m + q;
        const uint32_t slot = first ? k : h.n + (k - h.n) * m + q;
        const FuseCmd c = lds_uniform<FuseCmd>(&sg.cmd[k]);
        float* dst = nullptr;
        if (in_space) {
            const uint32_t ndims = first ? h.ndims : 1u;
            const uint32_t u0 = first ? c0 : 0u, u1 = first ? c1 : unit * VEC;
            if (c.op == FUSE_OP_DOT) {
                const uint32_t from = c.src & 0xFFu;
                if (!first && from != FUSE_SRC_MEMORY) member_dot_own<VEC>(c, q, staged[from * EW_BLOCK], r);
                else member_dot<VEC>(c, unit, r);
            } else {
                member_ew<VEC>(c, ndims, u0, u1, staged, first ? 1u : m, first ? 0 : (int)(h.n + q) - (int)(h.n * m), r);
            }
            staged[slot * EW_BLOCK] = r;
            dst = (float*)c.out + (ndims == 2 ? u0 * (uint32_t)c.os[0] + u1 * (uint32_t)c.os[1] : u1 * (uint32_t)c.os[0]);
        }
        where[slot * EW_BLOCK] = dst;
        if (c.fwd & FUSE_NEXT_IS_ZERO_PLUS) {
            // the pass that accumulates a gradient for the first time, `0 + g`: made here from the registers, for the
            // price of reading where it goes instead of a member's whole interpretation
            struct OutOf { void* out; const void* in[2]; int64_t os[2]; };
            const OutOf n = lds_uniform<OutOf>(&sg.cmd[k + 1]);
            const uint32_t slot2 = first ? slot + 1 : slot + m;
            float* dst2 = nullptr;
            if (dst) {
#pragma unroll
                for (int e = 0; e < VEC; ++e) r.v[e] = OpZeroPlus<float>{}(r.v[e]);
                staged[slot2 * EW_BLOCK] = r;
                const uint32_t u0 = first ? c0 : 0u, u1 = first ? c1 : unit * VEC;
                dst2 = (float*)n.out + (first && h.ndims == 2 ? u0 * (uint32_t)n.os[0] + u1 * (uint32_t)n.os[1] : u1 * (uint32_t)n.os[0]);
            }
            where[slot2 * EW_BLOCK] = dst2;
            ++k;
            ++it;
        }
        ++k;
        if (!first && k == h.n + h.nwide) { k = h.n; ++q; }
    }
    {
        // every member's output to memory, in member order (a later member may write where an earlier one did)
        for (uint32_t k0 = 0; k0 < slots; k0 += 4) {
            AVec<float, VEC> o[4];
            float* dst[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const uint32_t k = k0 + i < slots ? k0 + i : k0;
                o[i] = staged[k * EW_BLOCK];
                dst[i] = where[k * EW_BLOCK];
            }
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (k0 + i < slots && dst[i]) {
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
