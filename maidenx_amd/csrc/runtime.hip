// Device, memory, stream and status entry points of the backend.  They replace the
// cuda_malloc / cuda_free / cuda_memcpy_* / cuda_set_device / cuda_get_device family of
// crates/maidenx_cuda/src/lib.rs:39-117.
#include <cstdio>
#include <cstring>
#include <mutex>
#include <vector>

#include "mxh.hpp"

namespace mxh {

static std::mutex g_mu;
static std::mutex g_scratch_mu;
static int g_status = OK;
static int g_hip_err = 0;
static char g_what[256] = "ok";
static hipStream_t g_stream = nullptr;      // null = the device's default stream
static hipStream_t g_capture_stream = nullptr;   // created on first use, default priority
static hipStream_t g_saved_stream = nullptr;
static bool g_capturing = false;
// recording of a capture as a program (see program.hpp)
static bool g_prog_enabled = true;
static bool g_prog_ok = false;            // every launch of the open capture so far has a command
static bool g_prog_pending = false;       // a command was recorded and its launch not yet seen
static std::vector<ProgCmd> g_prog_cmds;
struct GraphExec {                        // what hip_graph_end_capture hands out
    hipGraphExec_t graph = nullptr;
    ProgCmd* cmds = nullptr;              // device copy of the program, when the capture is one
    uint32_t n = 0;
};
// A capture that called scratch() has the block's address baked into its graph or program: while such a capture is
// alive the block must not be freed, so a later growth retires it instead (freed with the last live capture).
static bool g_scratch_captured[16][2] = {{false}};
static int g_live_captures = 0;
static std::vector<void*> g_retired_scratch;
static void* g_scratch[16][2] = {{nullptr}};
static size_t g_scratch_bytes[16][2] = {{0}};

void set_status(int code, const char* what, int hip_err) {
    std::lock_guard<std::mutex> lk(g_mu);
    if (g_status != OK) return;   // keep the first error
    g_status = code;
    g_hip_err = hip_err;
    if (hip_err != 0)
        snprintf(g_what, sizeof(g_what), "%s: %s", what, hipGetErrorString((hipError_t)hip_err));
    else
        snprintf(g_what, sizeof(g_what), "%s", what);
}

hipStream_t stream() { return g_stream; }

bool prog_recording() { return g_capturing && g_prog_ok; }
void prog_record(uint32_t kid, unsigned grid, const void* args, size_t bytes) {
    if (!prog_recording()) return;
    if (bytes > PROG_ARG_BYTES || grid > PROG_MAX_GRID || g_prog_pending || g_prog_cmds.size() >= 65536) { g_prog_ok = false; return; }
    ProgCmd c;
    std::memset((void*)&c, 0, sizeof(c));
    c.kid = kid;
    c.grid = grid;
    std::memcpy(c.args, args, bytes);
    g_prog_cmds.push_back(c);
    g_prog_pending = true;
}
void prog_launch_seen() {
    if (!g_capturing) return;
    if (g_prog_pending) g_prog_pending = false;
    else g_prog_ok = false;               // a launch without a command: only the HIP graph can replay this capture
}

void* scratch(size_t bytes, int slot) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16 || slot < 0 || slot > 1) {
        set_status(ERR_INVALID, "scratch: bad device or slot");
        return nullptr;
    }
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    if (g_scratch_bytes[dev][slot] >= bytes) {
        if (g_capturing) g_scratch_captured[dev][slot] = true;
        return g_scratch[dev][slot];
    }
    if (g_capturing) {      // growing means a synchronise and a free, neither of which a capture allows
        set_status(ERR_INVALID, "scratch would have to grow during graph capture: run the sequence eagerly once first");
        return nullptr;
    }
    // grow: work already queued on the stream may still use the old block, so drain first
    if (g_scratch[dev][slot]) {
        (void)hipStreamSynchronize(g_stream);
        if (g_scratch_captured[dev][slot] && g_live_captures > 0) g_retired_scratch.push_back(g_scratch[dev][slot]);
        else (void)hipFree(g_scratch[dev][slot]);
        g_scratch_captured[dev][slot] = false;
        g_scratch[dev][slot] = nullptr;
        g_scratch_bytes[dev][slot] = 0;
    }
    size_t want = bytes < (32u << 20) ? (32u << 20) : bytes;
    void* p = nullptr;
    hipError_t e = hipMalloc(&p, want);
    if (e != hipSuccess) { set_status(ERR_OOM, "scratch: hipMalloc", (int)e); return nullptr; }
    g_scratch[dev][slot] = p;
    g_scratch_bytes[dev][slot] = want;
    return p;
}

static int* g_index_flag[16] = {nullptr};
static bool g_index_flag_used[16] = {false};

int* index_flag() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) { set_status(ERR_INVALID, "index flag: bad device"); return nullptr; }
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    if (!g_index_flag[dev]) {
        if (g_capturing) { set_status(ERR_INVALID, "the first index op of a device cannot run inside a graph capture"); return nullptr; }
        int* p = nullptr;
        hipError_t e = hipMalloc((void**)&p, 256);
        if (e == hipSuccess) e = hipMemset(p, 0, 256);
        if (e != hipSuccess) { set_status(ERR_OOM, "index flag: hipMalloc", (int)e); return nullptr; }
        g_index_flag[dev] = p;
    }
    g_index_flag_used[dev] = true;
    return g_index_flag[dev];
}

// Waits for the stream and folds a raised index flag of the current device into the status.
static void collect_index_flag() {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return;
    int* p;
    {
        std::lock_guard<std::mutex> lk(g_scratch_mu);
        if (!g_index_flag_used[dev] || g_capturing) return;
        g_index_flag_used[dev] = false;
        p = g_index_flag[dev];
    }
    int v = 0;
    if (hipStreamSynchronize(g_stream) != hipSuccess) return;
    if (g_capture_stream) (void)hipStreamSynchronize(g_capture_stream);
    if (hipMemcpy(&v, p, sizeof(int), hipMemcpyDeviceToHost) != hipSuccess) return;
    if (v != 0) {
        (void)hipMemset(p, 0, sizeof(int));
        set_status(ERR_INVALID, "index out of bounds in index_select / index_add_ / gather / scatter_add_ / bincount");
    }
}

}  // namespace mxh

using namespace mxh;

extern "C" {

int hip_set_device(int id) { return (int)hipSetDevice(id); }
int hip_get_device(int* id) { return (int)hipGetDevice(id); }
int hip_device_count(int* n) { return (int)hipGetDeviceCount(n); }

int hip_malloc(void** ptr, size_t bytes) {
    if (!ptr) return (int)hipErrorInvalidValue;
    if (bytes == 0) bytes = 1;
    hipError_t e = hipMalloc(ptr, bytes);
    return e == hipSuccess ? 0 : (e == hipErrorOutOfMemory ? ERR_OOM : (int)e);
}
int hip_free(void* ptr) { return (int)hipFree(ptr); }

// The copies are ordered after everything queued on the backend's stream and return when done.
int hip_memcpy_h2d(void* dst, const void* src, size_t bytes) {
    hipError_t e = hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, stream());
    if (e == hipSuccess) e = hipStreamSynchronize(stream());
    return (int)e;
}
int hip_memcpy_d2h(void* dst, const void* src, size_t bytes) {
    hipError_t e = hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, stream());
    if (e == hipSuccess) e = hipStreamSynchronize(stream());
    return (int)e;
}
int hip_memcpy_d2d(void* dst, const void* src, size_t bytes) {
    prog_launch_seen();
    return (int)hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, stream());
}

int hip_stream_create(void** s) { return (int)hipStreamCreateWithFlags((hipStream_t*)s, hipStreamNonBlocking); }
int hip_stream_destroy(void* s) { return (int)hipStreamDestroy((hipStream_t)s); }
int hip_stream_synchronize(void* s) { return (int)hipStreamSynchronize((hipStream_t)s); }
// Stream every later kernel and copy of the backend is queued on (null = default stream).
int hip_set_stream(void* s) { g_stream = (hipStream_t)s; return 0; }
void* hip_get_stream(void) { return (void*)g_stream; }
int hip_synchronize(void) {
    hipError_t e = hipStreamSynchronize(stream());
    if (e == hipSuccess && g_capture_stream && !g_capturing) e = hipStreamSynchronize(g_capture_stream);   // graph replays
    return (int)e;
}

// Events on the backend's stream, for timing kernels where they run.
int hip_event_create(void** ev) { return (int)hipEventCreate((hipEvent_t*)ev); }
int hip_event_destroy(void* ev) { return (int)hipEventDestroy((hipEvent_t)ev); }
int hip_event_record(void* ev) { return (int)hipEventRecord((hipEvent_t)ev, stream()); }
int hip_event_synchronize(void* ev) { return (int)hipEventSynchronize((hipEvent_t)ev); }
int hip_event_elapsed_ms(void* start, void* stop, float* ms) { return (int)hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop); }

// First error recorded since the last call (0 = none); reading it clears it.
int hip_get_last_status(void) {
    collect_index_flag();
    hipError_t e = hipGetLastError();
    std::lock_guard<std::mutex> lk(g_mu);
    if (g_status == OK && e != hipSuccess) {
        g_status = ERR_LAUNCH;
        g_hip_err = (int)e;
        snprintf(g_what, sizeof(g_what), "hip: %s", hipGetErrorString(e));
    }
    int s = g_status;
    g_status = OK;
    return s;
}
// Text of the error last returned by hip_get_last_status().
const char* hip_status_string(void) { return g_what; }


int hip_graph_begin_capture(void) {
    if (g_capturing) return (int)hipErrorInvalidValue;
    hipError_t e = hipDeviceSynchronize();
    if (e != hipSuccess) return (int)e;
    if (!g_capture_stream) {
        e = hipStreamCreate(&g_capture_stream);
        if (e != hipSuccess) return (int)e;
    }
    e = hipStreamBeginCapture(g_capture_stream, hipStreamCaptureModeThreadLocal);
    if (e != hipSuccess) return (int)e;
    g_saved_stream = g_stream;
    g_stream = g_capture_stream;
    g_capturing = true;
    g_prog_ok = g_prog_enabled;
    g_prog_pending = false;
    g_prog_cmds.clear();
    return 0;
}
int hip_graph_end_capture(void** graph_exec) {
    if (!g_capturing || !graph_exec) return (int)hipErrorInvalidValue;
    hipGraph_t graph = nullptr;
    hipError_t e = hipStreamEndCapture(g_capture_stream, &graph);
    g_stream = g_saved_stream;
    g_capturing = false;
    const bool as_program = g_prog_ok && !g_prog_pending && !g_prog_cmds.empty();
    if (e != hipSuccess) return (int)e;
    GraphExec* ge = new GraphExec();
    if (as_program) {
        // every launch of the capture has a command: replays are one launch of the interpreter
        (void)hipGraphDestroy(graph);
        const size_t bytes = g_prog_cmds.size() * sizeof(ProgCmd);
        e = hipMalloc((void**)&ge->cmds, bytes);
        if (e == hipSuccess) e = hipMemcpy(ge->cmds, g_prog_cmds.data(), bytes, hipMemcpyHostToDevice);
        if (e != hipSuccess) { if (ge->cmds) (void)hipFree(ge->cmds); delete ge; return (int)e; }
        ge->n = (uint32_t)g_prog_cmds.size();
    } else {
        e = hipGraphInstantiate(&ge->graph, graph, nullptr, nullptr, 0);
        (void)hipGraphDestroy(graph);
        if (e != hipSuccess) { delete ge; return (int)e; }
    }
    g_prog_cmds.clear();
    {
        std::lock_guard<std::mutex> lk(g_scratch_mu);
        ++g_live_captures;
    }
    *graph_exec = (void*)ge;
    return 0;
}
// 1 when the capture behind `graph_exec` replays as one interpreter launch, 0 when it is a HIP graph.
int hip_graph_is_program(void* graph_exec) { return graph_exec && ((GraphExec*)graph_exec)->cmds ? 1 : 0; }
// Whether later captures may become programs (default 1); returns the previous setting.
int hip_graph_set_programs(int enabled) {
    int was = g_prog_enabled ? 1 : 0;
    g_prog_enabled = enabled != 0;
    return was;
}
// Replays run on the capture stream, a blocking stream: work on the default stream orders with it.
int hip_graph_launch(void* graph_exec) {
    if (!graph_exec || !g_capture_stream || g_capturing) return (int)hipErrorInvalidValue;
    GraphExec* ge = (GraphExec*)graph_exec;
    if (ge->cmds) {
        prog_launch(ge->cmds, ge->n, (void*)g_capture_stream);
        return (int)hipGetLastError();
    }
    return (int)hipGraphLaunch(ge->graph, g_capture_stream);
}
int hip_graph_destroy(void* graph_exec) {
    if (!graph_exec) return 0;
    (void)hipStreamSynchronize(g_capture_stream);
    GraphExec* ge = (GraphExec*)graph_exec;
    hipError_t e = hipSuccess;
    if (ge->cmds) e = hipFree(ge->cmds);
    if (ge->graph) e = hipGraphExecDestroy(ge->graph);
    delete ge;
    {
        // the last live capture is gone: nothing refers to retired scratch blocks, or to the current ones, any more
        std::lock_guard<std::mutex> lk(g_scratch_mu);
        if (--g_live_captures <= 0) {
            g_live_captures = 0;
            for (void* p : g_retired_scratch) (void)hipFree(p);
            g_retired_scratch.clear();
            for (auto& dev : g_scratch_captured) dev[0] = dev[1] = false;
        }
    }
    return (int)e;
}

}  // extern "C"
