// Resident step programs: a whole capture of small f32 launches as ONE work-group that keeps its tensors in LDS.
//
// A training step on tensors of a few thousand elements (the README's Linear(3 -> 1) + MSE + SGD on 10000 rows) is
// two dozen dependent launches that together touch 200 KB.  Replayed as graph nodes or as fused chains they cost
// microseconds each - for dependencies, not for work: a result written by one kernel is read by the next through
// memory, and a work-group that waits for another pays a device-scope release.  When every launch of a capture is one
// the fused chains would take (f32 elementwise over at most two collapsed dims, the one-thread-per-output matmul, a row
// sum that one work-group does, the few-output long-reduction matmul, the fused MSE loss) and small, the capture is recorded as a list of
// commands instead, and a replay is ONE launch of ONE 512-thread work-group that
//   * keeps every tensor the commands write in LDS for as long as it is alive (a liveness plan made on the host from
//     the commands' operand ranges and from the caller's hints that a buffer was released, hip_buffer_discard): a
//     command's operand is a byte offset into the LDS arena or a device address, and both are reached through generic
//     pointers, so the reductions and small matmuls are the very device functions the eager kernels call;
//   * maps element u of an elementwise command to thread u mod 512, always: consecutive commands that meet each
//     other's data element for element need no barrier at all - a thread only re-reads what it wrote - and the host
//     puts a work-group barrier in front of the commands that do read across threads;
//   * can run the command list many times in one launch (hip_graph_launch_n): tensors that one pass hands to the next
//     (parameters) stay in LDS from the first pass to the last, and memory sees every live tensor once, at the end.
// Every command applies the same functor or calls the same device function as its eager kernel, in the same order of
// additions: the bytes are those of the separate launches.  Anything that does not fit (a launch of another kind, a
// tensor too large) hands the launches recorded so far to the fused chains and the capture goes on as before.
#pragma once
#include <cstddef>
#include <cstdint>
#include <functional>
#include <vector>

#include "fuse.hpp"

namespace mxh {

enum ResKind : uint32_t { RES_EW = 0, RES_DOT = 1, RES_ROW = 2, RES_TAILDOT = 3, RES_MSE = 4 };
constexpr uint32_t RES_BARRIER = 1u;          // ResCmd::flags: a work-group barrier before the command
constexpr uint32_t RES_VEC = 2u;              // elementwise / matmul producer: a unit is a 16-byte vector
constexpr uint32_t RES_FAST = 8u;             // elementwise: every operand is one scalar or walked linearly (step[] is valid)
constexpr uint32_t RES_TWO_IN = 1u << 7;      // elementwise: the functor takes two inputs
constexpr uint32_t RES_LDS_OUT = 1u << 4;     // operand 0 (the output), 1, 2 (inputs) lives in the arena: its pointer
constexpr uint32_t RES_LDS_IN0 = 1u << 5;     // field holds the byte offset
constexpr uint32_t RES_LDS_IN1 = 1u << 6;
constexpr unsigned RES_THREADS = 512;
constexpr int RES_UNROLL = 5;                 // units a thread has in flight (10000 elements are 2500 vectors: one round)
constexpr size_t RES_LDS_BYTES = (160u << 10) - 256;  // dynamic LDS of the work-group: the arena
constexpr size_t RES_MAX_REGION = 64u << 10;          // larger tensors stay in memory
constexpr size_t RES_INPUT_BYTES = 64u << 10;         // of the arena for copies of inputs that no command writes
// Elements one command may span: the hard limit, and the default of hip_graph_set_resident().  One work-group's
// instruction stream is what a command costs: about 0.7 us for up to 2048 elements (one vector a thread), 1.5 us for
// 10000 - where the fused chains, which spread a launch over ten work-groups, are ahead again.  The README step
// (Linear(3 -> 1) + MSE + SGD) on n rows, us per step here / as chains: n = 256 12.0 / 19.3, 1000 14.2 / 19.0, 2000 15.5 /
// 21.8, 3000 20.4 / 23.9, 5000 25.5 / 21.6, 10000 34.0 / 22.6 - the default keeps tensors of up to 8192 elements here.
constexpr size_t RES_MAX_ELEMS = 1u << 16;
constexpr size_t RES_DEFAULT_ELEMS = 8192;
constexpr uint32_t RES_MODE_LINEAR = 0, RES_MODE_SCALAR = 1, RES_MODE_2D = 2;

// The first 64 bytes are all an elementwise command in its fast form needs: one scalar load.
struct alignas(64) ResCmd {
    uint32_t kind, flags, sub, units;         // sub: elementwise: the functor's position in EwProgOps; tail stages: as recorded
    uint64_t p_out, p_in0, p_in1;             // the operands, resolved: byte offset into the arena (RES_LDS_*) or device address
    int32_t step[3];                          // RES_FAST: elements a unit advances operand k (0 = output) by; 0 = one scalar for all
    uint32_t payload[2];                      // RES_FAST: the functor's state
    uint32_t mode;                            // byte k: how operand k is addressed in the general form (RES_MODE_*)
    FastDiv div_inner;                        // elementwise over two dims: the inner extent; matmul producer: J
    uint32_t pad;
    alignas(16) unsigned char arg[FUSE_TAIL_ARG_BYTES];      // FuseCmd (RES_EW, RES_DOT), RowProgArgs, GemmArgs, MseArgs
};
static_assert(sizeof(ResCmd) == 192 && offsetof(ResCmd, mode) == 60, "the fast form is the first 64 bytes");

// One launch as the launch sites hand it to the open capture (runtime.hip), kept so that it can still be given to the
// fused chains, or launched, when the capture turns out not to be a resident program.
struct ResRecord {
    uint32_t kind = RES_EW;                   // or RES_DISCARD below
    uint32_t sub = 0;                         // tail stages: as fuse_record_tail()
    uint32_t tail_kind = 0;
    bool vec = false;
    uint32_t ndims = 1, dims[2] = {1, 1};
    size_t units = 0;                         // elementwise and matmul producer: vectors or elements of the space
    size_t outputs = 0;                       // matmul producer and tail stages: outputs
    alignas(16) unsigned char arg[FUSE_TAIL_ARG_BYTES];
    size_t arg_bytes = 0;
    int nin = 0;
    Extent out{0, 0}, in[2] = {{0, 0}, {0, 0}};
    std::function<void()> relaunch;           // set when the fused chains would refuse the launch: launches it for real
    bool chain_ok = true;                     // matmul producer: a chain may be offered it at all
};
constexpr uint32_t RES_DISCARD = 0xD15Cu;     // ResRecord::kind: the caller released [out.lo, out.hi)

struct ResProgram {
    std::vector<ResCmd> host_cmds;            // until res_upload()
    ResCmd* device_cmds = nullptr;
    uint32_t n_pro = 0, n_body = 0, n_epi = 0;
    uint32_t lds_bytes = 0;
    uint32_t in_lds = 0, barriers = 0;        // (for reporting) operands served from LDS, barriers per pass
};

// resident.hip: plans the records of a capture as a program, on the host (false: they cannot be one) ...
bool res_build(const std::vector<ResRecord>& recs, ResProgram& out);
// ... and puts it on the device (not while a stream capture is open: it allocates and copies).
bool res_upload(ResProgram& p);
// resident.hip: prologue, `passes` times the body, epilogue - one launch.
void res_launch(const ResProgram& p, uint32_t passes, void* stream);
void res_destroy(ResProgram& p);

}  // namespace mxh
