// Resident step programs (see resident.hpp): the interpreter kernel and the host-side planner.
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "elementwise.hpp"
#include "fuse.hpp"
#include "fuse_ops.hpp"
#include "gemm_small.hpp"
#include "loss.hpp"
#include "mxh.hpp"
#include "ops.hpp"
#include "reduce_row.hpp"
#include "resident.hpp"

namespace mxh {

// ---- the interpreter -------------------------------------------------------------------------------------------
// The command list does not change while the kernel runs: it is read through the constant address space, i.e. by scalar
// loads into scalar registers, whole commands at a time.
typedef const __attribute__((address_space(4))) ResCmd* ResCmdPtr;

template <class A>
__device__ __forceinline__ A res_args(ResCmdPtr c) {
    A a;
    __builtin_memcpy(&a, c->arg, sizeof(A));
    return a;
}
// A command's time is its instruction count: one wave issues an instruction every few nanoseconds however little it
// does, and a command is two to three hundred of them when every operand is addressed by the general rule.  So there
// are two forms.  The fast one serves operands that are one scalar or walked linearly (nearly all of a training step):
// 32-bit element offsets, `unit * step`.  The general one serves two collapsed dims with any strides.
//
// An operand is a device address or a byte offset into the arena, reached with the instructions of its own address
// space, chosen by a uniform branch: a generic ("flat") access to LDS waits for the vector memory path as well.  The
// reductions and the long-reduction matmuls are the eager kernels' device functions and take generic pointers.
typedef __attribute__((address_space(3))) unsigned char LdsByte;
typedef __attribute__((address_space(3))) float LdsFloat;
typedef __attribute__((address_space(1))) float MemFloat;
typedef float F4 __attribute__((ext_vector_type(4)));
struct ResOperand {
    uint64_t field;      // device address, or byte offset into the arena
    uint32_t lds;        // non-zero: in the arena
};
__device__ __forceinline__ float* res_ptr(uint64_t field, uint32_t in_lds, LdsByte* arena) {
    return in_lds ? (float*)(unsigned char*)(arena + (uint32_t)field) : (float*)field;
}

template <int VEC, class P>
__device__ __forceinline__ void res_load_from(P p, int64_t inner, float* dst) {
    if (VEC == 4 && inner == 1) {
        const F4 t = *(const F4 __attribute__((address_space(std::is_same<P, const LdsFloat*>::value ? 3 : 1)))*)p;
        dst[0] = t.x; dst[1] = t.y; dst[2] = t.z; dst[3] = t.w;
    } else if (inner == 0) {
        const float t = p[0];
#pragma unroll
        for (int e = 0; e < VEC; ++e) dst[e] = t;
    } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) dst[e] = p[(int64_t)e * inner];
    }
}
template <int VEC, class P>
__device__ __forceinline__ void res_store_to(P p, int64_t inner, const float* src) {
    if (VEC == 4 && inner == 1) {
        F4 t;
        t.x = src[0]; t.y = src[VEC > 1 ? 1 : 0]; t.z = src[VEC > 2 ? 2 : 0]; t.w = src[VEC > 3 ? 3 : 0];
        *(F4 __attribute__((address_space(std::is_same<P, LdsFloat*>::value ? 3 : 1)))*)p = t;
    } else {
#pragma unroll
        for (int e = 0; e < VEC; ++e) p[(int64_t)e * inner] = src[e];
    }
}
template <int VEC>
__device__ __forceinline__ void res_load(const ResOperand& o, LdsByte* arena, int64_t off, int64_t inner, float* dst) {
    if (o.lds) res_load_from<VEC>((const LdsFloat*)(arena + (uint32_t)o.field) + (int32_t)off, inner, dst);
    else res_load_from<VEC>((const MemFloat*)o.field + off, inner, dst);
}
template <int VEC>
__device__ __forceinline__ void res_store(const ResOperand& o, LdsByte* arena, int64_t off, int64_t inner, const float* src) {
    if (o.lds) res_store_to<VEC>((LdsFloat*)(arena + (uint32_t)o.field) + (int32_t)off, inner, src);
    else res_store_to<VEC>((MemFloat*)o.field + off, inner, src);
}

// ---- elementwise, fast form: unit u of the command belongs to thread u mod 512 - whatever the command, which is what
// lets dependent commands over one space follow each other without a barrier - and operand k's elements for it start at
// element u * step[k].  U units of a thread are in flight together; a thread without a unit repeats the last one's loads
// and stores nothing.
template <int VEC, int U, bool LONG>
__device__ __forceinline__ void res_ew_fast(ResCmdPtr c, uint32_t flags, uint32_t units, unsigned tid, LdsByte* arena) {
    const uint32_t op = c->sub;
    const ResOperand out{c->p_out, flags & RES_LDS_OUT}, in0{c->p_in0, flags & RES_LDS_IN0}, in1{c->p_in1, flags & RES_LDS_IN1};
    const int32_t so = c->step[0], s0 = c->step[1], s1 = c->step[2];
    const uint32_t payload[2] = {c->payload[0], c->payload[1]};
    const bool two = flags & RES_TWO_IN;
    for (uint32_t u0 = 0; u0 < units; u0 += U * RES_THREADS) {
        float a[U * VEC], b[U * VEC], r[U * VEC];
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const uint32_t u = u0 + j * RES_THREADS + tid, uc = u < units ? u : units - 1;
            res_load<VEC>(in0, arena, (int32_t)uc * s0, s0 != 0, a + j * VEC);
            if (two) res_load<VEC>(in1, arena, (int32_t)uc * s1, s1 != 0, b + j * VEC);
            else {
#pragma unroll
                for (int e = 0; e < VEC; ++e) b[j * VEC + e] = 0.0f;
            }
        }
        fuse_switch<U * VEC, LONG>(op, a, b, r, payload);
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const uint32_t u = u0 + j * RES_THREADS + tid;
            if (u < units) res_store<VEC>(out, arena, (int32_t)u * so, VEC == 4 ? 1 : so, r + j * VEC);
        }
    }
}

template <int VEC>
__device__ __attribute__((noinline)) void res_ew_fast_long(ResCmdPtr c, uint32_t flags, uint32_t units, unsigned tid, LdsByte* arena) {
    res_ew_fast<VEC, 1, true>(c, flags, units, tid, arena);
}

// ---- elementwise, general form: two collapsed dims, any strides (out of line, like the long functors: rare in a step,
// and inlined they cost every command registers)
__device__ __forceinline__ int64_t res_offset(uint32_t mode, uint32_t ndims, const int64_t (&s)[2], uint32_t e0, uint32_t c0, uint32_t c1) {
    if (mode == RES_MODE_SCALAR) return 0;
    if (mode == RES_MODE_LINEAR) return (int64_t)e0 * (ndims == 2 ? s[1] : s[0]);
    return (int64_t)c0 * s[0] + (int64_t)c1 * s[1];
}
template <int VEC, bool LONG>
__device__ __attribute__((noinline)) void res_ew_general(ResCmdPtr c, uint32_t flags, uint32_t units, unsigned tid, LdsByte* arena) {
    const FuseCmd f = res_args<FuseCmd>(c);
    FastDiv dv;
    dv.d = c->div_inner.d; dv.mul = c->div_inner.mul; dv.shift = c->div_inner.shift;
    const uint32_t mode = c->mode, ndims = f.ndims;
    const ResOperand out{c->p_out, flags & RES_LDS_OUT}, in0{c->p_in0, flags & RES_LDS_IN0}, in1{c->p_in1, flags & RES_LDS_IN1};
    const int64_t inner_o = ndims == 2 ? f.os[1] : f.os[0];
    const int64_t inner_0 = (mode >> 8 & 0xFFu) == RES_MODE_SCALAR ? 0 : (ndims == 2 ? f.is[0][1] : f.is[0][0]);
    const int64_t inner_1 = (mode >> 16 & 0xFFu) == RES_MODE_SCALAR ? 0 : (ndims == 2 ? f.is[1][1] : f.is[1][0]);
    for (uint32_t u = tid; u < units; u += RES_THREADS) {
        float a[VEC], b[VEC], r[VEC];
        const uint32_t e0 = u * VEC;
        uint32_t c0 = 0, c1 = e0;
        if (ndims == 2) fd_divmod(e0, dv, c0, c1);
        res_load<VEC>(in0, arena, res_offset(mode >> 8 & 0xFFu, ndims, f.is[0], e0, c0, c1), inner_0, a);
        if (f.nin > 1) res_load<VEC>(in1, arena, res_offset(mode >> 16 & 0xFFu, ndims, f.is[1], e0, c0, c1), inner_1, b);
        else {
#pragma unroll
            for (int e = 0; e < VEC; ++e) b[e] = 0.0f;
        }
        fuse_switch<VEC, LONG>(f.op, a, b, r, f.payload);
        res_store<VEC>(out, arena, res_offset(mode & 0xFFu, ndims, f.os, e0, c0, c1), inner_o, r);
    }
}
template <int VEC>
__device__ __forceinline__ void res_ew(ResCmdPtr c, uint32_t flags, uint32_t units, unsigned tid, LdsByte* arena) {
    const bool lng = is_long_op(c->sub);
    if (flags & RES_FAST) {
        // (the long functors - the libm restatements - are bound by their arithmetic: one unit at a time keeps their code
        // and their registers small; a command of one round has nothing to keep in flight either)
        if (lng) res_ew_fast_long<VEC>(c, flags, units, tid, arena);
        else if (units <= RES_THREADS) res_ew_fast<VEC, 1, false>(c, flags, units, tid, arena);
        else res_ew_fast<VEC, RES_UNROLL, false>(c, flags, units, tid, arena);
    } else {
        if (lng) res_ew_general<VEC, true>(c, flags, units, tid, arena);
        else res_ew_general<VEC, false>(c, flags, units, tid, arena);
    }
}

// The one-thread-per-output matmul over the flat space of its outputs: terms in ascending r, multiply and add unfused, as
// gemm_thread_body adds them.  A thread owns U units at a time and fetches Q terms of each before it adds any (terms past
// the end re-read the first of the chunk and are not added): one memory latency per chunk instead of one per term.
// Offsets are 32-bit element offsets (the planner checks that the operands allow it).
// U units a thread, Q terms of every one of them requested together
template <int VEC, int U, int Q, class PX, class PY>
__device__ __forceinline__ void res_dot_units(const FuseCmd& f, const FastDiv& dj, const ResOperand& out, PX X, PY Y, uint32_t units, unsigned tid, LdsByte* arena) {
    constexpr int N = U * VEC;
    const uint32_t R = f.dims[1];
    const uint32_t xi = (uint32_t)f.is[0][0], xr = (uint32_t)f.is[0][1], yr = (uint32_t)f.is[1][0], yj = (uint32_t)f.is[1][1];
    for (uint32_t u0 = 0; u0 < units; u0 += U * RES_THREADS) {
        uint32_t ox[N], oy[N];
        float acc[N];
#pragma unroll
        for (int n = 0; n < N; ++n) {
            const uint32_t u = u0 + (n / VEC) * RES_THREADS + tid;
            uint32_t i, j;
            fd_divmod((u < units ? u : 0u) * VEC + n % VEC, dj, i, j);      // a thread without a unit works on unit 0 (and stores nothing)
            ox[n] = i * xi;
            oy[n] = j * yj;
            acc[n] = 0.0f;
        }
        for (uint32_t q0 = 0; q0 < R; q0 += Q) {
            float xv[N][Q], yv[N][Q];
#pragma unroll
            for (int k = 0; k < Q; ++k) {
                const uint32_t q = q0 + k < R ? q0 + k : q0;
#pragma unroll
                for (int n = 0; n < N; ++n) {
                    xv[n][k] = X[ox[n] + q * xr];
                    yv[n][k] = Y[oy[n] + q * yr];
                }
            }
#pragma unroll
            for (int k = 0; k < Q; ++k)
                if (q0 + k < R) {
#pragma unroll
                    for (int n = 0; n < N; ++n) acc[n] = acc[n] + xv[n][k] * yv[n][k];
                }
        }
#pragma unroll
        for (int j = 0; j < U; ++j) {
            const uint32_t u = u0 + j * RES_THREADS + tid;
            if (u >= units) continue;
            res_store<VEC>(out, arena, (int64_t)u * VEC, 1, acc + j * VEC);
        }
    }
}
template <int VEC>
__device__ __forceinline__ void res_dot(ResCmdPtr c, uint32_t flags, uint32_t units, unsigned tid, LdsByte* arena) {
    const FuseCmd f = res_args<FuseCmd>(c);
    FastDiv dj;
    dj.d = c->div_inner.d; dj.mul = c->div_inner.mul; dj.shift = c->div_inner.shift;
    const ResOperand out{c->p_out, flags & RES_LDS_OUT};
    const uint64_t fx = c->p_in0, fy = c->p_in1;
    const bool lx = flags & RES_LDS_IN0, ly = flags & RES_LDS_IN1;
    const LdsFloat* xl = (const LdsFloat*)(arena + (uint32_t)fx);
    const LdsFloat* yl = (const LdsFloat*)(arena + (uint32_t)fy);
    const MemFloat* xm = (const MemFloat*)fx;
    const MemFloat* ym = (const MemFloat*)fy;
    // at most a unit a thread (a weight gradient's handful of outputs over a reduction of a few dozen terms): eight terms in
    // flight, so that the reduction costs an eighth of its memory latencies; else several units a thread, two terms each
    constexpr int UM = VEC == 4 ? 5 : 8;
    if (units <= RES_THREADS) {
        if (lx && ly) res_dot_units<VEC, 1, 8>(f, dj, out, xl, yl, units, tid, arena);
        else if (lx) res_dot_units<VEC, 1, 8>(f, dj, out, xl, ym, units, tid, arena);
        else if (ly) res_dot_units<VEC, 1, 8>(f, dj, out, xm, yl, units, tid, arena);
        else res_dot_units<VEC, 1, 8>(f, dj, out, xm, ym, units, tid, arena);
    } else {
        if (lx && ly) res_dot_units<VEC, UM, 2>(f, dj, out, xl, yl, units, tid, arena);
        else if (lx) res_dot_units<VEC, UM, 2>(f, dj, out, xl, ym, units, tid, arena);
        else if (ly) res_dot_units<VEC, UM, 2>(f, dj, out, xm, yl, units, tid, arena);
        else res_dot_units<VEC, UM, 2>(f, dj, out, xm, ym, units, tid, arena);
    }
}

template <int TPR>
__device__ __forceinline__ void res_row(uint32_t vec, const RowProgArgs& a, const float* in, float* out, unsigned tid, float* part) {
    // virtual 256-thread blocks side by side; the recorded launch had one block, so only the first has rows
    float* p = part + (tid / RB) * (RB / WAVE);
    if (vec) row_reduce_body<float, float, RSum, TPR, 4, false, 16>(in, out, a.rows, a.L, a.chunks, a.chunk_len, a.div, a.src_bf16, tid / RB, tid % RB, p);
    else row_reduce_body<float, float, RSum, TPR, 1, false, 16>(in, out, a.rows, a.L, a.chunks, a.chunk_len, a.div, a.src_bf16, tid / RB, tid % RB, p);
}
__device__ __forceinline__ void res_row_cmd(ResCmdPtr c, uint32_t flags, unsigned tid, LdsByte* arena, float* part) {
    const RowProgArgs a = res_args<RowProgArgs>(c);
    const float* in = res_ptr(c->p_in0, flags & RES_LDS_IN0, arena);
    float* out = res_ptr(c->p_out, flags & RES_LDS_OUT, arena);
    const uint32_t sub = c->sub, vec = sub & 1u, tpr = (sub >> 1) % 3;      // the reducer is RSum: nothing else is recorded
    if (tpr == 0) res_row<1>(vec, a, in, out, tid, part);
    else if (tpr == 1) res_row<WAVE>(vec, a, in, out, tid, part);
    else res_row<RB>(vec, a, in, out, tid, part);
}
__device__ __forceinline__ void res_taildot_cmd(ResCmdPtr c, uint32_t flags, unsigned tid, LdsByte* arena, float* part) {
    GemmArgs g = res_args<GemmArgs>(c);
    g.X = res_ptr(c->p_in0, flags & RES_LDS_IN0, arena);
    g.Y = res_ptr(c->p_in1, flags & RES_LDS_IN1, arena);
    g.out = res_ptr(c->p_out, flags & RES_LDS_OUT, arena);
    const unsigned outputs = g.I * g.J * g.batch;
    if (c->sub == 2) {      // one wave per output, the eight waves taking the outputs in turn
        for (unsigned o = tid / WAVE; o < outputs; o += RES_THREADS / WAVE) gemm_wavedot_body<float>(g, o, (int)(tid % WAVE), nullptr);
    } else if (c->sub == 1) {      // the eager path's choice, made on the host (fewer loads in flight than there: this kernel has half the registers)
        if (g.I * g.J <= 3) gemm_rowsdot_any<EW_BLOCK, 8>(g, tid, part);
        else gemm_rowsdot_any<EW_BLOCK, 5>(g, tid, part);
    }
    else for (unsigned o = 0; o < outputs; o += 4) {
        if (o) __syncthreads();              // the fold of the outputs before still reads `part`
        gemm_blockdot_body<float, EW_BLOCK, 4>(g, o, outputs, tid, part);
    }
}

// the fused MSE loss of at most 65536 elements: the eager kernel's one block, run by the first 256 threads
__device__ __forceinline__ void res_mse_cmd(ResCmdPtr c, uint32_t flags, unsigned tid, LdsByte* arena, float* part) {
    const MseArgs a = res_args<MseArgs>(c);
    const float* pred = res_ptr(c->p_in0, flags & RES_LDS_IN0, arena);
    const float* target = res_ptr(c->p_in1, flags & RES_LDS_IN1, arena);
    float* loss = res_ptr(c->p_out, flags & RES_LDS_OUT, arena);
    const bool active = tid < (unsigned)MSE_THREADS;
    const float sum = mse_block_sum(pred, target, (size_t)a.n, 0, 1, tid, part, active);
    if (tid == 0) loss[0] = OpDivScalar<float>{(float)(size_t)a.n}(sum);
}

// Dynamic LDS: the arena.
// `trace` (normally null): thread 0 notes the 100 MHz clock when each command of the first passes begins.
__global__ __launch_bounds__(RES_THREADS) void resident_kernel(const ResCmd* cmds, uint32_t n_pro, uint32_t n_body, uint32_t n_epi, uint32_t passes,
                                                               unsigned long long* trace, uint32_t trace_len) {
    extern __shared__ __attribute__((aligned(256))) unsigned char res_lds[];
    __shared__ float part[4 * RB / WAVE];
    LdsByte* arena = (LdsByte*)res_lds;
    const uint32_t total = n_pro + n_body * passes + n_epi;
    uint32_t k = 0, pass = 0;
    for (uint32_t step = 0; step < total; ++step) {
        // (the thread index is taken afresh by every command: left to itself the compiler computes everything any
        // command derives from it ahead of the loop and keeps it all alive - in spilled registers - around every command)
        unsigned tid = threadIdx.x;
        asm volatile("" : "+v"(tid));
        ResCmdPtr c = (ResCmdPtr)(cmds + k);
        const uint32_t kind = c->kind, flags = c->flags, units = c->units;
        if (trace && tid == 0 && step < trace_len) trace[step] = wall_clock64();
        if (flags & RES_BARRIER) __syncthreads();
        if (kind == RES_EW) {
            if (flags & RES_VEC) res_ew<4>(c, flags, units, tid, arena);
            else res_ew<1>(c, flags, units, tid, arena);
        } else if (kind == RES_DOT) {
            if (flags & RES_VEC) res_dot<4>(c, flags, units, tid, arena);
            else res_dot<1>(c, flags, units, tid, arena);
        } else if (kind == RES_ROW) {
            res_row_cmd(c, flags, tid, arena, part);
        } else if (kind == RES_MSE) {
            res_mse_cmd(c, flags, tid, arena, part);
        } else {
            res_taildot_cmd(c, flags, tid, arena, part);
        }
        ++k;
        if (k == n_pro + n_body && ++pass < passes) k = n_pro;
    }
    if (trace && threadIdx.x == 0 && total < trace_len) trace[total] = wall_clock64();
}

// ---- the planner -----------------------------------------------------------------------------------------------
namespace {

struct Region {
    uintptr_t lo = 0, hi = 0;
    bool written = false, live_in = false, candidate = false, pinned = false;
    uint32_t readers = 0;              // commands of a pass that read it
    int state = 0;                     // 0 as the pass found it, 1 defined by a write of this pass, 2 released
    bool in_lds = false;
    uint32_t slot_off = 0, slot_size = 0, lds_off = 0;
    size_t size() const { return hi - lo; }
};

struct Arena {
    std::vector<std::pair<uint32_t, uint32_t>> free_list;      // (offset, size), ascending
    explicit Arena(uint32_t capacity) : free_list{{0u, capacity}} {}
    uint32_t high = 0;
    bool get(uint32_t size, uint32_t& off) {
        for (size_t i = 0; i < free_list.size(); ++i) {
            if (free_list[i].second < size) continue;
            off = free_list[i].first;
            free_list[i].first += size;
            free_list[i].second -= size;
            if (free_list[i].second == 0) free_list.erase(free_list.begin() + (long)i);
            high = std::max(high, off + size);
            return true;
        }
        return false;
    }
    void put(uint32_t off, uint32_t size) {
        auto it = std::lower_bound(free_list.begin(), free_list.end(), std::make_pair(off, 0u));
        it = free_list.insert(it, {off, size});
        if (it + 1 != free_list.end() && it->first + it->second == (it + 1)->first) {
            it->second += (it + 1)->second;
            free_list.erase(it + 1);
        }
        if (it != free_list.begin() && (it - 1)->first + (it - 1)->second == it->first) {
            (it - 1)->second += it->second;
            free_list.erase(it);
        }
    }
};

// where an operand ended up, and how a thread walks it: two accesses with equal keys touch the same addresses from the
// same threads
struct AccessKey {
    int space = 0;                     // 0 memory, 1 arena, 2 the reductions' own LDS
    uintptr_t lo = 0, hi = 0;
    bool write = false;
    uint64_t uid = 0;                  // non-zero: read or written across threads, equal to nothing
    uintptr_t base = 0;
    int64_t s0 = 0, s1 = 0;
    uint32_t d0 = 0, d1 = 0, ndims = 0, vec = 0, units = 0;
    bool same_walk(const AccessKey& o) const {
        return uid == 0 && o.uid == 0 && space == o.space && base == o.base && s0 == o.s0 && s1 == o.s1 && d0 == o.d0 && d1 == o.d1 &&
               ndims == o.ndims && vec == o.vec && units == o.units;
    }
    bool overlaps(const AccessKey& o) const { return space == o.space && lo < o.hi && o.lo < hi; }
};

constexpr uint32_t kIdentity = (uint32_t)IndexOf<OpIdentity<float>, EwProgOps>::value;
constexpr uint32_t kFill = (uint32_t)IndexOf<OpFill<float>, EwProgOps>::value;
// inputs a record really reads: a fill names its own output as its input and ignores what it finds there
int inputs_of(const ResRecord& r) {
    if (r.kind == RES_EW && ((const FuseCmd*)r.arg)->op == kFill) return 0;
    return r.nin;
}

struct Planned {
    ResCmd cmd;
    AccessKey acc[4];
    int nacc = 0;
};

// operand k of a record: pointer field inside the argument block
void** operand_field(ResCmd& c, int k) {
    if (c.kind == RES_EW || c.kind == RES_DOT) {
        FuseCmd* f = (FuseCmd*)c.arg;
        return k == 0 ? &f->out : (void**)&f->in[k - 1];
    }
    if (c.kind == RES_ROW) {
        RowProgArgs* a = (RowProgArgs*)c.arg;
        return k == 0 ? &a->out : (void**)&a->in;
    }
    if (c.kind == RES_MSE) {
        MseArgs* a = (MseArgs*)c.arg;
        return k == 0 ? (void**)&a->loss : (k == 1 ? (void**)&a->pred : (void**)&a->target);
    }
    GemmArgs* g = (GemmArgs*)c.arg;
    return k == 0 ? &g->out : (k == 1 ? (void**)&g->X : (void**)&g->Y);
}

uint32_t mode_of(uint32_t ndims, const uint32_t* dims, const int64_t* s) {
    if (ndims == 1) return s[0] == 0 ? RES_MODE_SCALAR : RES_MODE_LINEAR;
    if (s[0] == 0 && s[1] == 0) return RES_MODE_SCALAR;
    if (s[0] == (int64_t)dims[1] * s[1]) return RES_MODE_LINEAR;
    return RES_MODE_2D;
}

Planned make_copy(uintptr_t dst, bool dst_lds, uintptr_t src, bool src_lds, size_t bytes, uintptr_t align_probe) {
    Planned p;
    std::memset((void*)&p.cmd, 0, sizeof(p.cmd));
    FuseCmd f;
    std::memset((void*)&f, 0, sizeof(f));
    const bool vec = bytes % 16 == 0 && align_probe % 16 == 0;
    f.out = (void*)dst;
    f.in[0] = (const void*)src;
    f.os[0] = 1;
    f.is[0][0] = 1;
    f.op = kIdentity;
    f.nin = 1;
    f.ndims = 1;
    f.dims[0] = (uint32_t)(bytes / 4);
    f.dims[1] = 1;
    f.nel = (uint32_t)(bytes / 4);
    p.cmd.kind = RES_EW;
    p.cmd.sub = kIdentity;
    p.cmd.flags = (vec ? RES_VEC : 0u) | (dst_lds ? RES_LDS_OUT : 0u) | (src_lds ? RES_LDS_IN0 : 0u);
    p.cmd.units = (uint32_t)(vec ? bytes / 16 : bytes / 4);
    p.cmd.div_inner = make_fastdiv(1);
    p.cmd.mode = 0;
    p.cmd.flags |= RES_FAST;
    p.cmd.p_out = dst;
    p.cmd.p_in0 = src;
    p.cmd.step[0] = p.cmd.step[1] = vec ? 4 : 1;
    std::memcpy(p.cmd.arg, &f, sizeof(f));
    for (int k = 0; k < 2; ++k) {
        AccessKey& a = p.acc[k];
        const uintptr_t at = k == 0 ? dst : src;
        a.space = (k == 0 ? dst_lds : src_lds) ? 1 : 0;
        a.lo = at;
        a.hi = at + bytes;
        a.write = k == 0;
        a.base = at;
        a.s0 = 1;
        a.d0 = (uint32_t)(bytes / 4);
        a.d1 = 1;
        a.ndims = 1;
        a.vec = vec ? 1 : 0;
        a.units = p.cmd.units;
    }
    p.nacc = 2;
    return p;
}

}  // namespace

bool res_build(const std::vector<ResRecord>& recs, ResProgram& out) {
    // 1. regions: the operand ranges of all commands, overlapping ones merged
    std::vector<std::pair<uintptr_t, uintptr_t>> spans;
    size_t ncmds = 0;
    for (const ResRecord& r : recs) {
        if (r.kind == RES_DISCARD) continue;
        ++ncmds;
        if (r.out.hi <= r.out.lo) return false;
        spans.push_back({r.out.lo, r.out.hi});
        for (int j = 0; j < inputs_of(r); ++j) {
            if (r.in[j].hi <= r.in[j].lo) return false;
            spans.push_back({r.in[j].lo, r.in[j].hi});
        }
    }
    if (ncmds == 0 || ncmds > 60000) return false;
    std::sort(spans.begin(), spans.end());
    std::vector<Region> regions;
    for (const auto& s : spans) {
        if (!regions.empty() && s.first < regions.back().hi) regions.back().hi = std::max(regions.back().hi, s.second);
        else {
            Region g;
            g.lo = s.first;
            g.hi = s.second;
            regions.push_back(g);
        }
    }
    auto region_of = [&](const Extent& e) -> Region& {
        size_t lo = 0, hi = regions.size();
        while (hi - lo > 1) {
            const size_t mid = (lo + hi) / 2;
            if (regions[mid].lo <= e.lo) lo = mid;
            else hi = mid;
        }
        return regions[lo];
    };
    auto release = [&](const Extent& e, auto&& fn) {
        for (Region& g : regions)
            if (g.lo >= e.lo && g.hi <= e.hi) fn(g);
    };
    // 2. what a pass needs from the pass before (or from memory, for the first): regions read before this pass defines them
    for (const ResRecord& r : recs) {
        if (r.kind == RES_DISCARD) {
            release(r.out, [](Region& g) { g.state = 2; });
            continue;
        }
        for (int j = 0; j < inputs_of(r); ++j) {
            Region& g = region_of(r.in[j]);
            if (g.state == 0) g.live_in = true;
            if (j == 0 || &g != &region_of(r.in[0])) ++g.readers;
        }
        Region& g = region_of(r.out);
        g.written = true;
        if (r.out.lo <= g.lo && r.out.hi >= g.hi) g.state = 1;
        else if (g.state == 0) g.live_in = true;      // a partial write: the rest may still be read
    }
    // 3. the arena: regions a pass inherits keep one place for the whole launch, the others get one per life
    Arena arena((uint32_t)RES_LDS_BYTES);
    std::vector<Region*> pinned;
    for (Region& g : regions) {
        g.candidate = g.written && g.size() <= RES_MAX_REGION && g.size() % 4 == 0 && g.lo % 4 == 0;
        g.slot_size = (uint32_t)(((g.lo % 256) + g.size() + 255) / 256 * 256);
        g.state = 0;
        if (g.candidate && g.live_in) pinned.push_back(&g);
    }
    std::sort(pinned.begin(), pinned.end(), [](const Region* a, const Region* b) { return a->size() < b->size(); });
    // Inputs that nothing writes and two or more commands of a pass read (the samples and targets of a training step): a
    // copy in the arena for the whole launch - one trip to memory per launch instead of one per reading command and
    // pass - as long as they leave most of the arena to the tensors the commands write.
    {
        std::vector<Region*> inputs;
        for (Region& g : regions)
            if (!g.written && g.live_in && g.readers >= 2 && g.size() <= RES_MAX_REGION && g.size() % 4 == 0 && g.lo % 4 == 0) inputs.push_back(&g);
        std::sort(inputs.begin(), inputs.end(), [](const Region* a, const Region* b) { return a->size() < b->size(); });
        size_t taken = 0;
        for (Region* g : inputs) {
            if (taken + g->slot_size > RES_INPUT_BYTES) break;
            taken += g->slot_size;
            g->candidate = true;
            pinned.push_back(g);
        }
    }
    for (Region* g : pinned) {
        if (!arena.get(g->slot_size, g->slot_off)) { g->candidate = false; continue; }
        g->pinned = g->in_lds = true;
        g->lds_off = g->slot_off + (uint32_t)(g->lo % 256);
    }
    std::vector<Planned> body;
    body.reserve(ncmds);
    uint64_t uid = 0;
    uint32_t served = 0;
    for (const ResRecord& r : recs) {
        if (r.kind == RES_DISCARD) {
            release(r.out, [&](Region& g) {
                g.state = 2;
                if (g.in_lds && !g.pinned) {
                    arena.put(g.slot_off, g.slot_size);
                    g.in_lds = false;
                }
            });
            continue;
        }
        Planned p;
        std::memset((void*)&p.cmd, 0, sizeof(p.cmd));
        p.cmd.kind = r.kind;
        p.cmd.sub = r.sub;
        p.cmd.flags = r.vec ? RES_VEC : 0u;
        p.cmd.div_inner = make_fastdiv(1);
        std::memcpy(p.cmd.arg, r.arg, r.arg_bytes);
        const bool ew = r.kind == RES_EW, dot = r.kind == RES_DOT;
        const int nin = inputs_of(r);
        if (ew || dot) {
            if (r.units == 0 || r.units > 0xFFFFFFFFull / 8) return false;
            p.cmd.units = (uint32_t)r.units;
            FuseCmd* f = (FuseCmd*)p.cmd.arg;
            if (ew) {
                f->ndims = r.ndims;
                f->dims[0] = r.dims[0];
                f->dims[1] = r.ndims == 2 ? r.dims[1] : 1;
                size_t nel = (size_t)f->dims[0] * f->dims[1];
                if (nel > RES_MAX_ELEMS || nel != r.units * (r.vec ? 4 : 1)) return false;
                f->nel = (uint32_t)nel;
                p.cmd.sub = f->op;
                if (r.ndims == 2) p.cmd.div_inner = make_fastdiv(r.dims[1]);
                p.cmd.mode = mode_of(r.ndims, f->dims, f->os) | mode_of(r.ndims, f->dims, f->is[0]) << 8 |
                             (f->nin > 1 ? mode_of(r.ndims, f->dims, f->is[1]) << 16 : 0u);
                if ((p.cmd.mode & 0xFFu) == RES_MODE_SCALAR && nel > 1) return false;      // every thread would write one element
            } else {
                if (r.units * (r.vec ? 4 : 1) > RES_MAX_ELEMS) return false;
                if (r.in[0].hi - r.in[0].lo >= (1ull << 31) || r.in[1].hi - r.in[1].lo >= (1ull << 31)) return false;      // 32-bit offsets
                p.cmd.div_inner = make_fastdiv(f->dims[0]);      // J
            }
        }
        // the output first defines (or redefines) its region: that is when it may move into the arena
        {
            Region& g = region_of(r.out);
            const bool covers = r.out.lo <= g.lo && r.out.hi >= g.hi;
            if (g.candidate && !g.in_lds && (covers || g.state == 2)) {
                // (inputs of this very command that live in the same region were read from where it was until now: a
                // region only moves when nothing of it is alive, or when it is overwritten whole - and then an input in it
                // would be read and overwritten by different rules; such a command keeps the region where it is)
                bool reads_it = false;
                for (int j = 0; j < nin; ++j) reads_it |= &region_of(r.in[j]) == &g;
                if (!reads_it && arena.get(g.slot_size, g.slot_off)) {
                    g.in_lds = true;
                    g.lds_off = g.slot_off + (uint32_t)(g.lo % 256);
                }
            }
            if (covers) g.state = 1;
        }
        // operands: where they are now, and how they are walked
        const Extent* ext[3] = {&r.out, &r.in[0], &r.in[1]};
        const uint32_t lds_flag[3] = {RES_LDS_OUT, RES_LDS_IN0, RES_LDS_IN1};
        for (int k = 0; k <= nin; ++k) {
            Region& g = region_of(*ext[k]);
            AccessKey& a = p.acc[p.nacc++];
            void** field = operand_field(p.cmd, k);
            uintptr_t at = (uintptr_t)*field;
            if (at < ext[k]->lo || at >= ext[k]->hi) return false;      // (negative strides are not recorded)
            if (g.in_lds) {
                a.space = 1;
                a.lo = g.lds_off + (ext[k]->lo - g.lo);
                a.hi = g.lds_off + (ext[k]->hi - g.lo);
                at = g.lds_off + (at - g.lo);
                *field = (void*)at;
                p.cmd.flags |= lds_flag[k];
                ++served;
            } else {
                a.space = 0;
                a.lo = ext[k]->lo;
                a.hi = ext[k]->hi;
            }
            (k == 0 ? p.cmd.p_out : k == 1 ? p.cmd.p_in0 : p.cmd.p_in1) = at;
            a.write = k == 0;
            a.base = at;
            if (ew || (dot && k == 0)) {
                const FuseCmd* f = (const FuseCmd*)p.cmd.arg;
                const int64_t* s = k == 0 ? f->os : f->is[k - 1];
                a.s0 = dot ? 1 : s[0];
                a.s1 = dot || r.ndims < 2 ? 0 : s[1];
                a.d0 = dot ? (uint32_t)(r.units * (r.vec ? 4 : 1)) : f->dims[0];
                a.d1 = dot ? 1 : f->dims[1];
                a.ndims = dot ? 1 : r.ndims;
                a.vec = r.vec ? 1 : 0;
                a.units = (uint32_t)r.units;
            } else {
                a.uid = ++uid;
            }
        }
        if (ew && nin == 0) {      // a fill: its (ignored) input is its output, wherever that is now
            FuseCmd* f = (FuseCmd*)p.cmd.arg;
            f->in[0] = f->out;
            p.cmd.p_in0 = p.cmd.p_out;
            if (p.cmd.flags & RES_LDS_OUT) p.cmd.flags |= RES_LDS_IN0;
        }
        if (ew) {
            // the fast form: every operand one scalar, or walked linearly with 32-bit offsets (vectors: along a unit stride)
            const FuseCmd* f = (const FuseCmd*)p.cmd.arg;
            const int vecw = r.vec ? 4 : 1;
            bool fast = true;
            for (int k = 0; k <= (int)f->nin && fast; ++k) {
                const uint32_t m = p.cmd.mode >> (8 * k) & 0xFFu;
                const int64_t* s = k == 0 ? f->os : f->is[k - 1];
                const int64_t inner = r.ndims == 2 ? s[1] : s[0];
                if (m == RES_MODE_SCALAR) p.cmd.step[k] = 0;
                else if (m == RES_MODE_LINEAR && inner > 0 && (inner == 1 || !r.vec) && inner * (int64_t)f->nel < (1ll << 31)) p.cmd.step[k] = (int32_t)(inner * vecw);
                else fast = false;
            }
            if (fast && p.cmd.step[0] != 0) p.cmd.flags |= RES_FAST;
            if (f->nin > 1) p.cmd.flags |= RES_TWO_IN;
            p.cmd.payload[0] = f->payload[0];
            p.cmd.payload[1] = f->payload[1];
        }
        // an elementwise command that writes where it also reads must meet its own data element for element
        if (ew)
            for (int k = 1; k <= nin; ++k)
                if (p.acc[k].overlaps(p.acc[0]) && !p.acc[k].same_walk(p.acc[0])) return false;
        if (r.kind == RES_ROW || r.kind == RES_TAILDOT || r.kind == RES_MSE) {      // the fold's own LDS is reused from command to command
            AccessKey& a = p.acc[p.nacc++];
            a.space = 2;
            a.lo = 0;
            a.hi = 1;
            a.write = true;
            a.uid = ++uid;
        }
        body.push_back(p);
    }
    // 4. prologue (what the first pass inherits) and epilogue (what is alive in the arena when the last pass ends)
    std::vector<Planned> all;
    uint32_t n_pro = 0, n_epi = 0;
    for (const Region* g : pinned)
        if (g->pinned) {
            all.push_back(make_copy(g->lds_off, true, g->lo, false, g->size(), g->lo));
            ++n_pro;
        }
    all.insert(all.end(), body.begin(), body.end());
    for (const Region& g : regions)
        if (g.in_lds && g.written && g.state != 2) {
            all.push_back(make_copy(g.lo, false, g.lds_off, true, g.size(), g.lo));
            ++n_epi;
        }
    // 5. barriers: in front of every command that meets, through other threads, what a command since the last barrier
    //    touched; always in front of a pass (it follows the pass before) and of the epilogue
    std::vector<AccessKey> pending;
    uint32_t barriers = 0;
    for (size_t i = 0; i < all.size(); ++i) {
        Planned& p = all[i];
        bool need = i == n_pro || i == n_pro + body.size();
        for (int k = 0; k < p.nacc && !need; ++k)
            for (const AccessKey& e : pending)
                if (p.acc[k].overlaps(e) && (p.acc[k].write || e.write) && !p.acc[k].same_walk(e)) { need = true; break; }
        if (need) {
            p.cmd.flags |= RES_BARRIER;
            pending.clear();
            if (i >= n_pro && i < n_pro + body.size()) ++barriers;
        }
        for (int k = 0; k < p.nacc; ++k) pending.push_back(p.acc[k]);
    }
    out.host_cmds.resize(all.size());
    for (size_t i = 0; i < all.size(); ++i) out.host_cmds[i] = all[i].cmd;
    out.device_cmds = nullptr;
    out.n_pro = n_pro;
    out.n_body = (uint32_t)body.size();
    out.n_epi = n_epi;
    out.lds_bytes = std::max<uint32_t>(arena.high, 256);
    out.in_lds = served;
    out.barriers = barriers;
    return true;
}

bool res_upload(ResProgram& p) {
    // more than 64 KB of LDS has to be allowed once per device
    static bool attr_set[64] = {false};
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess) { (void)hipGetLastError(); return false; }
    if (device < 0 || device >= 64 || !attr_set[device]) {
        hipError_t e = hipFuncSetAttribute((const void*)resident_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)RES_LDS_BYTES);
        if (e != hipSuccess) { (void)hipGetLastError(); return false; }
        if (device >= 0 && device < 64) attr_set[device] = true;
    }
    ResCmd* dev = nullptr;
    const size_t bytes = p.host_cmds.size() * sizeof(ResCmd);
    if (bytes == 0 || hipMalloc((void**)&dev, bytes) != hipSuccess) { (void)hipGetLastError(); return false; }
    if (hipMemcpy(dev, p.host_cmds.data(), bytes, hipMemcpyHostToDevice) != hipSuccess) {
        (void)hipGetLastError();
        (void)hipFree(dev);
        return false;
    }
    p.device_cmds = dev;
    p.host_cmds.clear();
    p.host_cmds.shrink_to_fit();
    return true;
}

void res_launch(const ResProgram& p, uint32_t passes, void* stream_) {
    if (!p.device_cmds || passes == 0) return;
    // MXH_RESIDENT_TRACE in the environment: the first launch of the process is timed command by command (and waited for)
    static bool trace_wanted = getenv("MXH_RESIDENT_TRACE") != nullptr;
    if (trace_wanted) {
        trace_wanted = false;
        const uint32_t len = p.n_pro + 2 * p.n_body + p.n_epi + 1;
        unsigned long long* dev = nullptr;
        std::vector<unsigned long long> t(len, 0);
        if (hipMalloc((void**)&dev, len * 8) == hipSuccess) {
            (void)hipMemset(dev, 0, len * 8);
            hipLaunchKernelGGL(resident_kernel, dim3(1), dim3(RES_THREADS), p.lds_bytes, (hipStream_t)stream_, p.device_cmds, p.n_pro, p.n_body, p.n_epi,
                               passes, dev, len);
            (void)hipStreamSynchronize((hipStream_t)stream_);
            (void)hipMemcpy(t.data(), dev, len * 8, hipMemcpyDeviceToHost);
            (void)hipFree(dev);
            std::vector<ResCmd> cmds(p.n_pro + p.n_body + p.n_epi);
            (void)hipMemcpy(cmds.data(), p.device_cmds, cmds.size() * sizeof(ResCmd), hipMemcpyDeviceToHost);
            for (uint32_t i = 0; i + 1 < len && t[i + 1]; ++i) {
                const uint32_t k = i < p.n_pro + p.n_body ? i : (passes > 1 ? p.n_pro + (i - p.n_pro - p.n_body) % p.n_body : i);
                const ResCmd& c = cmds[k < cmds.size() ? k : 0];
                fprintf(stderr, "[resident] step %3u cmd %3u kind %u op %4u units %6u flags %02x : %6.2f us\n", i, k, c.kind,
                        c.kind <= RES_DOT ? ((const FuseCmd*)c.arg)->op : c.sub, c.units, c.flags, (double)(t[i + 1] - t[i]) * 0.01);
            }
            return;
        }
    }
    hipLaunchKernelGGL(resident_kernel, dim3(1), dim3(RES_THREADS), p.lds_bytes, (hipStream_t)stream_, p.device_cmds, p.n_pro, p.n_body, p.n_epi, passes,
                       (unsigned long long*)nullptr, 0u);
    MXH_HIP(hipGetLastError());
}

void res_destroy(ResProgram& p) {
    if (p.device_cmds) (void)hipFree(p.device_cmds);
    p.device_cmds = nullptr;
}

}  // namespace mxh
