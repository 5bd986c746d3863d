// Fused chains of small launches inside a capture.
//
// A captured training step on small tensors is a few dozen dependent launches that each compute for well under a
// microsecond; replayed as graph nodes they cost 2 to 4 us apiece however small, because each node waits for the one
// before.  While a capture is open (and cannot be a whole-capture program, see program.hpp) such launches are not
// launched: they join the open CHAIN, which becomes ONE kernel node with two phases.
//
// Parallel phase - members over one shared index space, every thread owning one vector (or element) of it:
//   * an f32 elementwise launch over a collapsed space of at most two dims joins when it iterates over the same space in
//     the same form and every overlap with the earlier members is element for element (same base, same strides): each
//     thread then only ever re-reads what it wrote itself, and no ordering between threads is needed;
//   * a small matmul of the one-thread-per-output kind (a reduction of at most 16 terms) joins as a producer over the
//     flat space of its outputs; its operands are read across threads, so they may not overlap anything the chain's
//     earlier members write, nor may a later member write them;
//   * the backward pass of the fused MSE loss joins as an elementwise member of two inputs; the one value every thread
//     reads besides (the gradient of the loss) is held to the rule of a matmul's operands.
//   A second, WIDE space of m times as many units (m = 2..4) may follow the first: the thread that owns unit v of the
//   first space owns units m v .. m v + m - 1 of the wide one, and takes them in m rounds after the members of the first
//   space.  A wide member may therefore read what its OWN thread wrote there: the outer product [N,1] x [1,m] (a matmul
//   producer of one term, the input gradient of a layer with one output feature) whose left operand is, row for row, a
//   first-space member's output takes its rows idx / m - the thread's own - from that member's staged output.  Apart
//   from that a wide member touches nothing a first-space member writes and writes nothing one reads, and among
//   themselves wide members keep the rule above.  Once a wide member has joined, the first space takes no more members.
// Serial phase ("tail") - stages run in order by the work-group that finishes the parallel phase last (every group
// publishes its writes, then draws a ticket; the last ticket continues, the others exit, nobody waits):
//   * elementwise launches of at most 256 elements (a bias, a 3-element weight, a loss), any shapes, any overlaps;
//   * a row reduction that one work-group does in the eager path as well ([10000] -> [] sums);
//   * a matmul with a handful of outputs and a long reduction (the weight gradient of a 3-feature layer);
//   * the fused MSE loss of at most 65536 elements (one work-group in the eager path as well).
//   A stage is the same device code as its eager kernel, so results are the bytes of the separate launches.  A tail
//   stage may depend on anything before it in stream order.  A parallel member that arrives after tail stages were
//   queued is hoisted over them when it neither reads what they write nor writes what they read or write.
// The chain is closed by the next thing queued on the stream, by a launch that does not fit, or by the end of the
// capture.  Every output is still written.
#pragma once
#include <cstddef>
#include <cstdint>
#include <functional>

#include "mxh.hpp"

namespace mxh {

constexpr int FUSE_MAX_CMDS = 16;          // members of the parallel phase (staging slots: a wide member takes wide_m)
constexpr int FUSE_MAX_WIDE = 4;           // most units of the wide space per unit of the first
constexpr int FUSE_MAX_TAIL = 12;          // stages of the serial phase
constexpr uint32_t FUSE_OP_DOT = 0xD07u;   // FuseCmd::op of a matmul producer (the other values index EwProgOps)
// FuseCmd::op of the fused MSE loss's backward pass (loss.hpp): out = 0 + ((g / nel) * 2) * (in0 - in1), where g is the
// f32 the payload's 8 bytes point to (read by every thread; a null pointer stands for 1) and nel the element count
constexpr uint32_t FUSE_OP_MSE_BACKWARD = 0xB5Eu;
constexpr int FUSE_TAIL_ARG_BYTES = 112;
constexpr uint32_t FUSE_TICKETS = 1024;    // ticket slots per device

struct FuseCmd {
    void* out;
    const void* in[2];
    int64_t os[2];            // element strides of the output over the (at most two) collapsed dims
    int64_t is[2][2];         // the same for each input; FUSE_OP_DOT: {output row, reduction} of X, {reduction, output column} of Y
    uint32_t op;              // position of the functor in EwProgOps, FUSE_OP_DOT or FUSE_OP_MSE_BACKWARD
    uint32_t nin;
    uint32_t fwd;             // bit j: input j is, element for element, what the previous member wrote (taken from registers);
                              // FUSE_NEXT_IS_ZERO_PLUS: the member after this one is `0 + this one's output`, made along with it
    uint32_t ndims;           // the member's own space: only read in the tail
    uint32_t dims[2];         // FUSE_OP_DOT: {output columns, reduction length}
    uint32_t nel;
    // Byte j: where input j comes from when it is not forwarded.  Parallel phase: the number of the earlier member
    // whose output it is element for element (read from that member's staged output), or FUSE_SRC_MEMORY.  Tail: the
    // number of the earlier stage whose mirrored output holds it, FUSE_SRC_MEMORY (nothing in the tail writes it: it is
    // fetched when the tail starts) or FUSE_SRC_MEMORY_LATE (read from memory when the stage runs).
    uint32_t src;
    uint32_t payload[2];      // the functor's state (a scalar constant), bit for bit
};
constexpr uint32_t FUSE_NEXT_IS_ZERO_PLUS = 1u << 8;
constexpr uint32_t FUSE_SRC_MEMORY = 0xFFu, FUSE_SRC_MEMORY_LATE = 0xFEu;
enum TailKind : uint32_t { TAIL_EW = 0, TAIL_ROW_REDUCE = 1, TAIL_DOT = 2, TAIL_MSE = 3 };
struct TailCmd {
    uint32_t kind;
    uint32_t sub;             // TAIL_ROW_REDUCE: the instantiation number of row_prog_sub(); TAIL_DOT: 1 = the rows form, 2 = a wave per output
    uint32_t sync;            // before this stage: 0 nothing, 1 a barrier that orders LDS, 2 one that also waits for memory
    uint32_t fwd;             // TAIL_EW: as FuseCmd::fwd, against the stage before
    int32_t moff[2];          // TAIL_EW, input from a mirror: element offset of the input's base from that stage's output
    uint32_t mirrored;        // the stage's outputs (at most 256, contiguous) are also kept in LDS for later stages
    uint32_t pad;
    alignas(8) unsigned char arg[FUSE_TAIL_ARG_BYTES];      // FuseCmd, RowProgArgs, GemmArgs or MseArgs
};
static_assert(sizeof(FuseCmd) <= FUSE_TAIL_ARG_BYTES, "a tail stage holds an elementwise member");
struct alignas(16) FuseGroup {
    uint32_t n, ndims, vec;   // vec: every member moves 16-byte vectors along the inner dim
    uint32_t ntail;
    uint32_t dims[2];
    FastDiv div_inner;
    size_t nvec;              // vectors (vec) or elements per member
    uint32_t* ticket;         // zero between launches: counts the work-groups that have finished the parallel phase
    uint32_t prefetch;        // bit 2k+j: input j of tail stage k is fetched from memory when the tail starts
    uint32_t blocks;          // work-groups of the launch
    uint32_t nwide;           // members of the wide space: cmd[n .. n + nwide); n + nwide * wide_m staging slots in all
    uint32_t wide_m;          // units of the wide space per unit of the first
    uint32_t wide_nvec;       // units of the wide space (= wide_m * nvec)
    uint32_t pad[1];
    alignas(16) FuseCmd cmd[FUSE_MAX_CMDS];
    alignas(16) TailCmd tail[FUSE_MAX_TAIL];
};
static_assert(sizeof(FuseCmd) % 16 == 0 && sizeof(TailCmd) % 16 == 0, "the kernel copies whole 16-byte pieces of the members in use");
static_assert(sizeof(FuseGroup) <= 4096, "the chain travels as kernel arguments");

// byte range an operand of a recorded launch touches
struct Extent {
    uintptr_t lo, hi;
    bool overlaps(const Extent& o) const { return lo < o.hi && o.lo < hi; }
};

// fuse.hip: one launch of the chain on `stream`.
void fuse_launch(const FuseGroup& g, void* stream);
// fuse.hip: the current device's FUSE_TICKETS ticket slots (device memory, all zero); null when they cannot be located
uint32_t* fuse_tickets();
// runtime.hip: a graph capture is being recorded
bool capture_open();
// runtime.hip: offer a launch to the open chain; true = taken (the caller must not launch).
bool fuse_record(const FuseCmd& c, uint32_t ndims, const uint32_t* dims, bool vec, size_t nvec, size_t elem_bytes);
// a one-thread-per-output f32 matmul: x, y are the extents of its operands
// `relaunch`: launches the product for real; needed for products a chain refuses (at most 256 outputs, or - chain_ok
// false - a reduction of more than 16 terms) and a resident step program takes
bool fuse_record_dot(const FuseCmd& c, size_t outputs, const Extent& x, const Extent& y, std::function<void()> relaunch = {}, bool chain_ok = true);
// the backward pass of the fused MSE loss (c.op = FUSE_OP_MSE_BACKWARD, contiguous operands of c.nel elements):
// grad_loss is the one f32 every thread reads
bool fuse_record_mse_backward(const FuseCmd& c, bool vec, size_t nvec, const Extent& grad_loss);
// a tail stage with its argument block; in[0..nin) / out: the byte ranges it reads and writes (out: `outputs` contiguous
// f32 values)
bool fuse_record_tail(uint32_t kind, uint32_t sub, const void* arg, size_t arg_bytes, const Extent* in, int nin, const Extent& out, size_t outputs);
// a capture that holds a launch the interpreter has no command for can only be a HIP graph: say so before offering that
// launch to the chain (which only takes launches once the capture cannot be a program)
void prog_abandon();

}  // namespace mxh
