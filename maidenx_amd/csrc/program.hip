// Interpreter of recorded programs: one work-group runs a list of small-kernel commands in order.
//
// Every command names a kernel body (elementwise functor and form, row reduction, the two small matmul
// kernels) and carries the argument block its launch site would have passed.  The work-group's 1024 threads
// act as four virtual 256-thread blocks side by side (or one 1024-thread block), looping over the command's
// virtual grid.  Commands are separated by a work-group barrier, which also orders their global memory
// accesses: all waves of a work-group share one vector L1.  The command list is read through the constant
// address space - it does not change while the kernel runs - so argument blocks arrive as scalar loads.
#include "elementwise.hpp"
#include "gemm_small.hpp"
#include "mxh.hpp"
#include "ops.hpp"
#include "reduce_row.hpp"

namespace mxh {

typedef const __attribute__((address_space(4))) ProgCmd* ConstCmdPtr;

// the argument block of a command, copied out of the constant address space
template <class A>
__device__ __forceinline__ A load_args(ConstCmdPtr c) {
    A a;
    __builtin_memcpy(&a, c->args, sizeof(A));
    return a;
}

template <class Op, int VEC>
__device__ __forceinline__ void run_ew(ConstCmdPtr c, unsigned tid) {
    // the iteration space stays where it is (it is indexed by run-time dims); pointers and functor are copied
    typedef const __attribute__((address_space(4))) EwProgArgs<Op> Args;
    Args* a = (Args*)c->args;
    EwPtrs<Op::NIN> p;
    __builtin_memcpy(&p, &a->p, sizeof(p));
    Op op;
    __builtin_memcpy(&op, &a->op, sizeof(op));
    const size_t n = a->nvec;
    const unsigned grid = c->grid;
    for (unsigned b0 = 0; b0 < grid; b0 += PROG_THREADS / EW_BLOCK)
        ew_nd_body<Op, VEC>(a->sp, p, n, op, b0 + tid / EW_BLOCK, tid % EW_BLOCK);
}

template <int I>
__device__ __forceinline__ void dispatch_ew(uint32_t sub, ConstCmdPtr c, unsigned tid) {
    if constexpr (I < EwProgOps::size) {
        if ((sub >> 1) == (uint32_t)I) {
            using Op = typename TypeAt<I, EwProgOps>::type;
            constexpr int VEC = 16 / (sizeof(typename Op::In) > sizeof(typename Op::Out) ? sizeof(typename Op::In) : sizeof(typename Op::Out));
            if (sub & 1u) run_ew<Op, VEC>(c, tid);
            else run_ew<Op, 1>(c, tid);
        } else {
            dispatch_ew<I + 1>(sub, c, tid);
        }
    }
}

template <class R, int TPR, int VEC>
__device__ __forceinline__ void run_row(ConstCmdPtr c, unsigned tid, float* lds) {
    const RowProgArgs a = load_args<RowProgArgs>(c);
    const unsigned grid = c->grid;
    const float* in = (const float*)a.in;
    float* out = (float*)a.out;
    const size_t rows = a.rows, L = a.L, chunk_len = a.chunk_len;
    const unsigned chunks = a.chunks;
    const float div = a.div;
    const bool src_bf16 = a.src_bf16;
    float* part = lds + (tid / RB) * (RB / WAVE);
    for (unsigned b0 = 0; b0 < grid; b0 += PROG_THREADS / RB) {
        row_reduce_body<float, float, R, TPR, VEC>(in, out, rows, L, chunks, chunk_len, div, src_bf16, b0 + tid / RB, tid % RB, part);
        if constexpr (TPR > WAVE) __syncthreads();      // `part` is written again by the next round
    }
}
template <class R, int TPR>
__device__ __forceinline__ void run_row_vec(uint32_t vec, ConstCmdPtr c, unsigned tid, float* lds) {
    if (vec) run_row<R, TPR, 4>(c, tid, lds);
    else run_row<R, TPR, 1>(c, tid, lds);
}
template <class R>
__device__ __forceinline__ void run_row_tpr(uint32_t tpr, uint32_t vec, ConstCmdPtr c, unsigned tid, float* lds) {
    if (tpr == 0) run_row_vec<R, 1>(vec, c, tid, lds);
    else if (tpr == 1) run_row_vec<R, WAVE>(vec, c, tid, lds);
    else run_row_vec<R, RB>(vec, c, tid, lds);
}


__global__ __launch_bounds__(PROG_THREADS) void program_kernel(const ProgCmd* cmds, uint32_t n) {
    __shared__ float lds[PROG_THREADS / WAVE];
    const unsigned tid = threadIdx.x;
    for (uint32_t k = 0; k < n; ++k) {
        ConstCmdPtr c = (ConstCmdPtr)(cmds + k);
        const uint32_t kid = c->kid, family = kid >> 16, sub = kid & 0xFFFFu;
        if (family == PF_EW) {
            dispatch_ew<0>(sub, c, tid);
        } else if (family == PF_ROW_REDUCE) {
            const uint32_t vec = sub & 1u, tpr = (sub >> 1) % 3, red = (sub >> 1) / 3;
            if (red == 0) run_row_tpr<RSum>(tpr, vec, c, tid, lds);
            else if (red == 1) run_row_tpr<RMax>(tpr, vec, c, tid, lds);
            else run_row_tpr<RMin>(tpr, vec, c, tid, lds);
        } else if (family == PF_GEMM_THREAD) {
            const GemmArgs g = load_args<GemmArgs>(c);
            const unsigned grid = c->grid;
            for (unsigned b0 = 0; b0 < grid; b0 += PROG_THREADS / GB) gemm_thread_body<float>(g, b0 + tid / GB, tid % GB);
        } else if (family == PF_GEMM_ROWSDOT) {
            const GemmArgs g = load_args<GemmArgs>(c);
            gemm_rowsdot_any<256>(g, tid, lds);
        } else if (family == PF_GEMM_BLOCKDOT) {
            const GemmArgs g = load_args<GemmArgs>(c);
            const unsigned grid = c->grid;
            for (unsigned b = 0; b < grid; ++b) {
                gemm_blockdot_body<float, 256>(g, b, grid, tid, lds);      // a program command reads at most PROG_MAX_ELEMS: the short form
                __syncthreads();
            }
        }
        __syncthreads();      // the next command may read what this one wrote
    }
}

void prog_launch(const ProgCmd* device_cmds, uint32_t n, void* stream_) {
    hipLaunchKernelGGL(program_kernel, dim3(1), dim3(PROG_THREADS), 0, (hipStream_t)stream_, device_cmds, n);
    MXH_HIP(hipGetLastError());
}

}  // namespace mxh
