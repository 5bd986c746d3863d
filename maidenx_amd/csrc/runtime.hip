// Device, memory, stream and status entry points of the backend.  They replace the
// cuda_malloc / cuda_free / cuda_memcpy_* / cuda_set_device / cuda_get_device family of
// crates/maidenx_cuda/src/lib.rs:39-117.
#include <cstdio>
#include <cstring>
#include <mutex>
#include <thread>
#include <vector>

#include "fuse.hpp"
#include "mxh.hpp"

namespace mxh {

static std::mutex g_mu;
static std::mutex g_scratch_mu;
static std::recursive_mutex g_api_mu;       // held by every entry point for its whole duration (ApiGuard)
static std::thread::id g_capture_owner;     // the thread that opened the capture, while g_capturing
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
// fused runs of elementwise launches inside a capture (see fuse.hpp)
static bool g_fuse_enabled = true;
static FuseGroup g_fuse;                  // the open group (n == 0: none)
static size_t g_fuse_elem_bytes = 4;
static uint32_t g_fused_launches = 0, g_fuse_nodes = 0;     // of the open capture
struct GraphExec {                        // what hip_graph_end_capture hands out
    hipGraphExec_t graph = nullptr;
    ProgCmd* cmds = nullptr;              // device copy of the program, when the capture is one
    uint32_t n = 0;
    uint32_t fused_launches = 0, fuse_nodes = 0;
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

ApiGuard::ApiGuard() : ok(true) {
    g_api_mu.lock();
    if (g_capturing && g_capture_owner != std::this_thread::get_id()) {
        ok = false;
        set_status(ERR_INVALID, "another host thread has a graph capture open: calls from this thread are refused until it ends");
    }
}
ApiGuard::~ApiGuard() { g_api_mu.unlock(); }

static void fuse_flush() {
    if (g_fuse.n == 0) return;
    fuse_launch(g_fuse, (void*)g_capture_stream);
    ++g_fuse_nodes;
    g_fuse.n = 0;
}

// Every launch and copy of the library asks for the stream right before it queues something: an open group of fused
// launches has to run before that.
hipStream_t stream() {
    if (g_capturing && g_fuse.n) fuse_flush();
    return g_stream;
}

// byte range an operand touches
static void operand_range(const void* base, const int64_t* strides, uint32_t ndims, const uint32_t* dims, size_t esz, uintptr_t& lo, uintptr_t& hi) {
    size_t span = 0;
    for (uint32_t d = 0; d < ndims; ++d) span += (size_t)(dims[d] - 1) * (size_t)strides[d];
    lo = (uintptr_t)base;
    hi = lo + (span + 1) * esz;
}
static bool same_mapping(const void* a, const int64_t* sa, const void* b, const int64_t* sb, uint32_t ndims) {
    if (a != b) return false;
    for (uint32_t d = 0; d < ndims; ++d)
        if (sa[d] != sb[d]) return false;
    return true;
}

bool fuse_record(const FuseCmd& c, uint32_t ndims, const uint32_t* dims, bool vec, size_t nvec, size_t elem_bytes) {
    // only once the capture cannot be a whole-capture program any more (that path launches for real)
    if (!g_capturing || !g_fuse_enabled || g_prog_ok || ndims < 1 || ndims > 2) return false;
    for (uint32_t d = 0; d < ndims; ++d)
        if (c.os[d] < 0 || c.is[0][d] < 0 || (c.nin > 1 && c.is[1][d] < 0)) return false;
    // at most one block's worth of elements, one per thread: such members form groups of their own, in which a barrier
    // between members orders everything (any shapes, any overlaps)
    size_t nel = 1;
    for (uint32_t d = 0; d < ndims; ++d) nel *= dims[d];
    const bool tiny = nel <= 256;
    if (tiny) {
        if (!(g_fuse.n > 0 && g_fuse.tiny && g_fuse.n < (uint32_t)FUSE_MAX_CMDS)) {
            fuse_flush();
            g_fuse.tiny = 1;
            g_fuse.vec = 0;
            g_fuse.ndims = 1;
            g_fuse.nvec = 256;
            g_fuse.dims[0] = 256;
            g_fuse.dims[1] = 1;
            g_fuse.div_inner = make_fastdiv(1);
            g_fuse_elem_bytes = elem_bytes;
        }
        FuseCmd& slot = g_fuse.cmd[g_fuse.n++];
        slot = c;
        slot.fwd = 0;            // the forwarded registers belong to another member's thread layout
        slot.ndims = ndims;
        slot.dims[0] = dims[0];
        slot.dims[1] = ndims == 2 ? dims[1] : 1;
        slot.nel = (uint32_t)nel;
        ++g_fused_launches;
        return true;
    }
    if (g_fuse.n > 0 && g_fuse.tiny) fuse_flush();
    const bool fits = g_fuse.n > 0 && g_fuse.n < (uint32_t)FUSE_MAX_CMDS && g_fuse.ndims == ndims && g_fuse.vec == (vec ? 1u : 0u) &&
                      g_fuse.nvec == nvec && g_fuse.dims[0] == dims[0] && (ndims == 1 || g_fuse.dims[1] == dims[1]) && g_fuse_elem_bytes == elem_bytes;
    bool join = fits;
    if (join) {
        // every overlap with an earlier member must be element for element, so that a thread only meets its own data
        uintptr_t olo, ohi;
        operand_range(c.out, c.os, ndims, dims, elem_bytes, olo, ohi);
        for (uint32_t k = 0; k < g_fuse.n && join; ++k) {
            const FuseCmd& e = g_fuse.cmd[k];
            uintptr_t lo, hi;
            operand_range(e.out, e.os, ndims, dims, elem_bytes, lo, hi);
            // read after write, and write after write
            for (uint32_t j = 0; j < c.nin && join; ++j) {
                uintptr_t ilo, ihi;
                operand_range(c.in[j], c.is[j], ndims, dims, elem_bytes, ilo, ihi);
                if (ilo < hi && lo < ihi && !same_mapping(c.in[j], c.is[j], e.out, e.os, ndims)) join = false;
            }
            if (olo < hi && lo < ohi && !same_mapping(c.out, c.os, e.out, e.os, ndims)) join = false;
            // write after read
            for (uint32_t j = 0; j < e.nin && join; ++j) {
                uintptr_t ilo, ihi;
                operand_range(e.in[j], e.is[j], ndims, dims, elem_bytes, ilo, ihi);
                if (olo < ihi && ilo < ohi && !same_mapping(c.out, c.os, e.in[j], e.is[j], ndims)) join = false;
            }
        }
    }
    if (!join) {
        fuse_flush();
        g_fuse.tiny = 0;
        g_fuse.ndims = ndims;
        g_fuse.vec = vec ? 1u : 0u;
        g_fuse.nvec = nvec;
        g_fuse.dims[0] = dims[0];
        g_fuse.dims[1] = ndims == 2 ? dims[1] : 1;
        g_fuse.div_inner = make_fastdiv(g_fuse.dims[ndims - 1]);
        g_fuse_elem_bytes = elem_bytes;
    }
    FuseCmd& slot = g_fuse.cmd[g_fuse.n];
    slot = c;
    slot.fwd = 0;
    if (g_fuse.n > 0) {
        const FuseCmd& prev = g_fuse.cmd[g_fuse.n - 1];
        for (uint32_t j = 0; j < c.nin; ++j)
            if (same_mapping(c.in[j], c.is[j], prev.out, prev.os, ndims)) slot.fwd |= 1u << j;
    }
    ++g_fuse.n;
    ++g_fused_launches;
    return true;
}

bool capture_open() { return g_capturing; }
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
        if (g_capture_stream) (void)hipStreamSynchronize(g_capture_stream);     // replays queued there use the block as well
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

int hip_set_device(int id) { MXH_API_INT; return (int)hipSetDevice(id); }
int hip_get_device(int* id) { MXH_API_INT; return (int)hipGetDevice(id); }
int hip_device_count(int* n) { return (int)hipGetDeviceCount(n); }

int hip_malloc(void** ptr, size_t bytes) {
    MXH_API_INT;
    if (!ptr) return (int)hipErrorInvalidValue;
    if (bytes == 0) bytes = 1;
    hipError_t e = hipMalloc(ptr, bytes);
    return e == hipSuccess ? 0 : (e == hipErrorOutOfMemory ? ERR_OOM : (int)e);
}
int hip_free(void* ptr) { MXH_API_INT; return (int)hipFree(ptr); }

// The copies are ordered after everything queued on the backend's stream and return when done.
int hip_memcpy_h2d(void* dst, const void* src, size_t bytes) {
    MXH_API_INT;
    hipError_t e = hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, stream());
    if (e == hipSuccess) e = hipStreamSynchronize(stream());
    return (int)e;
}
int hip_memcpy_d2h(void* dst, const void* src, size_t bytes) {
    MXH_API_INT;
    hipError_t e = hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, stream());
    if (e == hipSuccess) e = hipStreamSynchronize(stream());
    return (int)e;
}
int hip_memcpy_d2d(void* dst, const void* src, size_t bytes) {
    MXH_API_INT;
    prog_launch_seen();
    return (int)hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, stream());
}

int hip_stream_create(void** s) { return (int)hipStreamCreateWithFlags((hipStream_t*)s, hipStreamNonBlocking); }
int hip_stream_destroy(void* s) { return (int)hipStreamDestroy((hipStream_t)s); }
int hip_stream_synchronize(void* s) { return (int)hipStreamSynchronize((hipStream_t)s); }
// Stream every later kernel and copy of the backend is queued on (null = default stream).
int hip_set_stream(void* s) {
    MXH_API_INT;
    // replays queued on the capture stream were ordered with the old stream only
    if (g_capture_stream && (hipStream_t)s != g_stream) (void)hipStreamSynchronize(g_capture_stream);
    g_stream = (hipStream_t)s;
    return 0;
}
void* hip_get_stream(void) { std::lock_guard<std::recursive_mutex> lk(g_api_mu); return (void*)g_stream; }
int hip_synchronize(void) {
    MXH_API_INT;
    hipError_t e = hipStreamSynchronize(stream());
    if (e == hipSuccess && g_capture_stream && !g_capturing) e = hipStreamSynchronize(g_capture_stream);   // graph replays
    return (int)e;
}

// Events on the backend's stream, for timing kernels where they run.
int hip_event_create(void** ev) { return (int)hipEventCreate((hipEvent_t*)ev); }
int hip_event_destroy(void* ev) { return (int)hipEventDestroy((hipEvent_t)ev); }
int hip_event_record(void* ev) { MXH_API_INT; return (int)hipEventRecord((hipEvent_t)ev, stream()); }
int hip_event_synchronize(void* ev) { return (int)hipEventSynchronize((hipEvent_t)ev); }
int hip_event_elapsed_ms(void* start, void* stop, float* ms) { return (int)hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop); }

// First error recorded since the last call (0 = none); reading it clears it.
int hip_get_last_status(void) {
    std::lock_guard<std::recursive_mutex> api(g_api_mu);     // not refused during another thread's capture: it queues nothing
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
    MXH_API_INT;
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
    g_capture_owner = std::this_thread::get_id();
    g_prog_ok = g_prog_enabled;
    g_prog_pending = false;
    g_prog_cmds.clear();
    g_fuse.n = 0;
    g_fused_launches = g_fuse_nodes = 0;
    return 0;
}
int hip_graph_end_capture(void** graph_exec) {
    MXH_API_INT;
    if (!g_capturing || !graph_exec) return (int)hipErrorInvalidValue;
    fuse_flush();
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
    ge->fused_launches = g_fused_launches;
    ge->fuse_nodes = g_fuse_nodes;
    {
        std::lock_guard<std::mutex> lk(g_scratch_mu);
        ++g_live_captures;
    }
    *graph_exec = (void*)ge;
    return 0;
}
// 1 when the capture behind `graph_exec` replays as one interpreter launch, 0 when it is a HIP graph.
int hip_graph_is_program(void* graph_exec) { return graph_exec && ((GraphExec*)graph_exec)->cmds ? 1 : 0; }
// Elementwise launches of the capture that were fused into groups, and (nodes != NULL) the kernel nodes they became.
int hip_graph_fused_launches(void* graph_exec, int* nodes) {
    if (!graph_exec) return 0;
    if (nodes) *nodes = (int)((GraphExec*)graph_exec)->fuse_nodes;
    return (int)((GraphExec*)graph_exec)->fused_launches;
}
// Whether later captures may fuse runs of elementwise launches (default 1); returns the previous setting.
int hip_graph_set_fusion(int enabled) {
    std::lock_guard<std::recursive_mutex> api(g_api_mu);
    int was = g_fuse_enabled ? 1 : 0;
    g_fuse_enabled = enabled != 0;
    return was;
}
// Whether later captures may become programs (default 1); returns the previous setting.
int hip_graph_set_programs(int enabled) {
    std::lock_guard<std::recursive_mutex> api(g_api_mu);
    int was = g_prog_enabled ? 1 : 0;
    g_prog_enabled = enabled != 0;
    return was;
}
// A replay is ordered with the library's eager work, which shares its tensors and both scratch slots.  With the default
// (null) stream it runs on the capture stream: that one is a blocking stream, and the null stream orders with blocking
// streams in both directions.  Once the caller has set a stream of its own (hip_stream_create gives non-blocking
// ones, which order with nothing) the replay is queued on that stream, behind the eager work and ahead of what follows.
int hip_graph_launch(void* graph_exec) {
    MXH_API_INT;
    if (!graph_exec || !g_capture_stream || g_capturing) return (int)hipErrorInvalidValue;
    GraphExec* ge = (GraphExec*)graph_exec;
    hipStream_t s = g_stream ? g_stream : g_capture_stream;
    if (ge->cmds) {
        prog_launch(ge->cmds, ge->n, (void*)s);
        return (int)hipGetLastError();
    }
    return (int)hipGraphLaunch(ge->graph, s);
}
int hip_graph_destroy(void* graph_exec) {
    MXH_API_INT;
    if (!graph_exec) return 0;
    (void)hipStreamSynchronize(g_capture_stream);
    if (g_stream) (void)hipStreamSynchronize(g_stream);      // replays run there once the caller has set a stream
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
