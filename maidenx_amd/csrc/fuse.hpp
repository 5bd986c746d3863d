// Fused runs of elementwise launches inside a capture.
//
// A captured training step is mostly runs of elementwise kernels over one index space, each reading what the one
// before wrote.  Replayed as graph nodes they cost 1.6-1.8 us apiece however small.  While a capture is open (and
// cannot be a whole-capture program, see program.hpp), an f32 elementwise launch over a collapsed space of at most
// two dims is not launched: it joins the open group when it iterates over the same space in the same form and every
// overlap with the group's earlier members is element for element (same base, same strides) - then each thread
// only ever re-reads what it wrote itself, and no ordering between threads is needed.  The group is closed by the
// next thing queued on the stream, by a launch that does not fit, or by the end of the capture, and becomes ONE
// kernel node that applies the members in order per element.  Every output is still written; results are the bytes
// of the separate launches.
// Members of at most 256 elements (a bias, a 3-element weight, a loss) need none of this care: a group of those is
// run by a single work-group with a barrier between members, whatever their shapes and however they overlap.
#pragma once
#include <cstddef>
#include <cstdint>

#include "mxh.hpp"

namespace mxh {

constexpr int FUSE_MAX_CMDS = 16;
struct FuseCmd {
    void* out;
    const void* in[2];
    int64_t os[2];            // element strides of the output over the (at most two) collapsed dims
    int64_t is[2][2];         // the same for each input
    uint32_t op;              // position of the functor in EwProgOps
    uint32_t nin;
    uint32_t fwd;             // bit j: input j is, element for element, what the previous member wrote (taken from registers)
    uint32_t ndims;           // the member's own space: only read in a tiny group
    uint32_t dims[2];
    uint32_t nel;
    uint32_t reserved;
    uint32_t payload[2];      // the functor's state (a scalar constant), bit for bit
};
struct alignas(16) FuseGroup {
    uint32_t n, ndims, vec;   // vec: every member moves 16-byte vectors along the inner dim
    uint32_t tiny;            // 1: members of at most one block's worth of elements each, any shapes, run by ONE block with a barrier between them
    uint32_t dims[2];
    FastDiv div_inner;
    size_t nvec;              // vectors (vec) or elements per member
    FuseCmd cmd[FUSE_MAX_CMDS];
};

// fuse.hip: one launch of the group on `stream`.
void fuse_launch(const FuseGroup& g, void* stream);
// runtime.hip: offers a launch to the open group; true = taken (the caller must not launch).
bool fuse_record(const FuseCmd& c, uint32_t ndims, const uint32_t* dims, bool vec, size_t nvec, size_t elem_bytes);

}  // namespace mxh
