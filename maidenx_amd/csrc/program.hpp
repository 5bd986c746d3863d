// Recorded programs of small kernels.
//
// A training step on small tensors is a few dozen dependent launches of kernels that each run for well
// under a microsecond; replayed from a HIP graph such a step still costs about 3 us per kernel node.  While
// a capture is open, the launch sites of the kernels listed below also append a command (kernel id, virtual
// grid, argument block) to a host list.  When every launch of the capture was one of them and small, the
// capture is turned into a "program": the commands go to device memory once, and a replay is ONE launch of
// an interpreter (a single work-group of 1024 threads) that runs the commands in order with a work-group
// barrier between them - the same kernel bodies, called with virtual block and thread indices.  Anything
// else in the capture (a tensor of more than a few thousand elements, a kernel without a body here, a copy)
// leaves the HIP graph as the replay path.
#pragma once
#include <cstddef>
#include <cstdint>

namespace mxh {

constexpr int PROG_ARG_BYTES = 496;
constexpr unsigned PROG_THREADS = 1024;       // threads of the interpreter's work-group
// One work-group has one CU's bandwidth (about 150 GB/s) and one CU's ALUs: only very small commands are cheaper here
// than as graph nodes.  Measured per command, mul_f32: 1.0 / 1.8 / 1.9 us in a program against 1.6 / 1.75 / 1.8 us
// as a HIP graph node for 256 / 4096 / 10000 elements - so a command may have one virtual block (4096 elements in
// vector form) and a capture is a program only if all of its launches are that small.
constexpr unsigned PROG_MAX_GRID = 1;         // virtual 256-thread blocks one command may have
constexpr size_t PROG_MAX_ELEMS = 4096;       // elements a reduction or small matmul command may read
struct alignas(16) ProgCmd {
    uint32_t kid;                             // family << 16 | instantiation
    uint32_t grid;                            // virtual blocks
    uint32_t pad[2];
    unsigned char args[PROG_ARG_BYTES];
};
static_assert(sizeof(ProgCmd) == 512, "one command is 512 bytes");

enum ProgFamily : uint32_t { PF_EW = 1, PF_ROW_REDUCE = 2, PF_GEMM_THREAD = 3, PF_GEMM_BLOCKDOT = 4, PF_GEMM_ROWSDOT = 5 };
inline uint32_t prog_kid(uint32_t family, uint32_t sub) { return (family << 16) | sub; }

// Host side (runtime.hip).  prog_recording(): a capture is open and still replayable by the interpreter.
bool prog_recording();
// A launch the interpreter has a body for.  Call it before the launch itself.
void prog_record(uint32_t kid, unsigned grid, const void* args, size_t bytes);
// Every launch or stream operation of the library reports here (MXH_LAUNCH_CHECK does it for kernels):
// one that was not preceded by prog_record() makes the capture a plain HIP graph.
void prog_launch_seen();

// Defined in program.hip: one launch of the interpreter over n commands in device memory.
void prog_launch(const ProgCmd* device_cmds, uint32_t n, void* stream);

}  // namespace mxh
