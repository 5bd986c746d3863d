// Device, memory, stream and status entry points of the backend.  They replace the
// cuda_malloc / cuda_free / cuda_memcpy_* / cuda_set_device / cuda_get_device family of
// crates/maidenx_cuda/src/lib.rs:39-117.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <algorithm>
#include <functional>
#include <mutex>
#include <thread>
#include <vector>

#include "ew_registry.hpp"
#include "fuse.hpp"
#include "mxh.hpp"
#include "resident.hpp"

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
// a capture as a resident step program (see resident.hpp): launches are kept here instead of being launched
static size_t g_res_elems = RES_DEFAULT_ELEMS;       // elements a kept launch may span; 0: no resident programs
static bool g_res_ok = false;             // every launch of the open capture so far is one the program can hold
static bool g_res_spilling = false;       // the kept launches are being handed on to the fused chains
static std::vector<ResRecord> g_res;
struct GraphExec {                        // what hip_graph_end_capture hands out
    hipGraphExec_t graph = nullptr;
    ResProgram res;                       // the capture as a resident step program (res.device_cmds != null)
    ProgCmd* cmds = nullptr;              // device copy of the program, when the capture is one
    uint32_t n = 0;
    uint32_t fused_launches = 0, fuse_nodes = 0;
};
// A capture that called scratch() has the block's address baked into its graph or program: while such a capture is
// alive the block must not be freed, so a later growth retires it instead (freed with the last live capture).
static bool g_scratch_captured[16][3] = {{false}};
static int g_live_captures = 0;
static std::vector<void*> g_retired_scratch;
static void* g_scratch[16][3] = {{nullptr}};
static size_t g_scratch_bytes[16][3] = {{0}};

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

// ---- the open chain of fused launches (see fuse.hpp) ----------------------------------------------------------
// What the recorded members read and write, for the checks a newcomer has to pass.
struct ParMember {
    Extent out, in[2];
    bool across[2];           // input j is read across threads (a matmul operand): it can never be "the same mapping"
    Extent extra{0, 0};       // one more range read across threads (the scalar of FUSE_OP_MSE_BACKWARD); empty: none
};
struct TailStage {
    Extent out, in[2];
    int nin;
    bool late[2];             // input j is read from memory when the stage runs (not fetched when the tail starts, not from a mirror)
    bool mirrored;            // the outputs are also kept in LDS
};
static ParMember g_par[FUSE_MAX_CMDS];
static TailStage g_tail[FUSE_MAX_TAIL];
static uint32_t g_lds_from = 0, g_mem_from = 0;      // first tail stage not yet ordered by a barrier (of LDS / that waits for memory)
static uint32_t* g_tickets[16] = {nullptr};       // per device: the ticket slots of fuse.hip
static bool g_tickets_ready = false;              // ... known for the device of the open capture
static uint32_t g_next_ticket = 0;

static void fuse_flush() {
    if (g_fuse.n == 0 && g_fuse.ntail == 0) return;
    int dev = 0;
    (void)hipGetDevice(&dev);
    // Chains queued on one stream run one after the other, and each leaves its ticket at zero, so sharing would do;
    // rotating over the slots keeps two captures that a caller replays on two streams at once apart as well.
    g_fuse.ticket = g_tickets[dev] + (g_next_ticket++ % FUSE_TICKETS);
    // MXH_CHAIN_TRACE in the environment: the shape of every chain as it is queued
    static const bool trace = getenv("MXH_CHAIN_TRACE") != nullptr;
    if (trace) {
        fprintf(stderr, "chain: %u members over %zu %s, %u wide x %u, tail stages of kind", g_fuse.n, g_fuse.nvec, g_fuse.vec ? "vectors" : "elements", g_fuse.nwide,
                g_fuse.wide_m);
        for (uint32_t k = 0; k < g_fuse.ntail; ++k) fprintf(stderr, " %u", g_fuse.tail[k].kind);
        fprintf(stderr, "\n");
    }
    fuse_launch(g_fuse, (void*)g_capture_stream);
    ++g_fuse_nodes;
    g_fuse.n = 0;
    g_fuse.nwide = g_fuse.wide_m = g_fuse.wide_nvec = 0;
    g_fuse.ntail = 0;
    g_lds_from = g_mem_from = 0;
}

// Every launch and copy of the library asks for the stream right before it queues something: an open chain of fused
// launches has to run before that.
static void res_spill();
hipStream_t stream() {
    if (g_capturing && g_res_ok && !g_res_spilling) res_spill();      // something is about to be launched for real
    if (g_capturing && (g_fuse.n || g_fuse.ntail)) fuse_flush();
    return g_stream;
}

// byte range an operand touches
static Extent operand_range(const void* base, const int64_t* strides, uint32_t ndims, const uint32_t* dims, size_t esz) {
    size_t span = 0;
    for (uint32_t d = 0; d < ndims; ++d) span += (size_t)(dims[d] - 1) * (size_t)strides[d];
    return Extent{(uintptr_t)base, (uintptr_t)base + (span + 1) * esz};
}
static bool same_mapping(const void* a, const int64_t* sa, const void* b, const int64_t* sb, uint32_t ndims) {
    if (a != b) return false;
    for (uint32_t d = 0; d < ndims; ++d)
        if (sa[d] != sb[d]) return false;
    return true;
}
static bool fuse_accepting() { return g_capturing && g_fuse_enabled && !g_prog_ok && g_tickets_ready; }

// A newcomer to the parallel phase against the tail stages already queued: it runs before them, so it may not read
// what they write nor write what they read or write.
static bool clear_of_tail(const ParMember& m, uint32_t nin) {
    for (uint32_t k = 0; k < g_fuse.ntail; ++k) {
        const TailStage& t = g_tail[k];
        if (m.out.overlaps(t.out)) return false;
        for (int j = 0; j < t.nin; ++j)
            if (m.out.overlaps(t.in[j])) return false;
        for (uint32_t j = 0; j < nin; ++j)
            if (m.in[j].overlaps(t.out)) return false;
        if (m.extra.overlaps(t.out)) return false;
    }
    return true;
}
// ... and against the earlier members of the parallel phase: every overlap must be element for element, so that a
// thread only meets its own data.  `wide`: the newcomer belongs to the wide space, where this holds against the wide
// members; of the first space's members it may only read an output as the rows of a one-term product (`own_rows`: the
// member it does that with, or -1), and otherwise shares no byte with what they write, nor writes what they read.
static bool clear_of_members(const FuseCmd& c, const ParMember& m, uint32_t ndims, bool wide, int own_rows) {
    const uint32_t members = g_fuse.n + g_fuse.nwide;
    for (uint32_t k = 0; k < members; ++k) {
        const FuseCmd& e = g_fuse.cmd[k];
        const ParMember& pe = g_par[k];
        if (wide && k < g_fuse.n) {
            for (uint32_t j = 0; j < c.nin; ++j)
                if (m.in[j].overlaps(pe.out) && !(j == 0 && (int)k == own_rows)) return false;
            if (m.out.overlaps(pe.out) || m.out.overlaps(pe.extra) || m.extra.overlaps(pe.out)) return false;
            for (uint32_t j = 0; j < e.nin; ++j)
                if (m.out.overlaps(pe.in[j])) return false;
            continue;
        }
        // read after write
        for (uint32_t j = 0; j < c.nin; ++j)
            if (m.in[j].overlaps(pe.out) && (m.across[j] || !same_mapping(c.in[j], c.is[j], e.out, e.os, ndims))) return false;
        // write after write
        if (m.out.overlaps(pe.out) && !same_mapping(c.out, c.os, e.out, e.os, ndims)) return false;
        // write after read
        for (uint32_t j = 0; j < e.nin; ++j)
            if (m.out.overlaps(pe.in[j]) && (pe.across[j] || !same_mapping(c.out, c.os, e.in[j], e.is[j], ndims))) return false;
        // the range every thread reads: nothing of the chain may write it, before or after
        if (m.extra.overlaps(pe.out) || m.out.overlaps(pe.extra)) return false;
    }
    return true;
}
static void open_space(uint32_t ndims, const uint32_t* dims, bool vec, size_t nvec, size_t elem_bytes) {
    g_fuse.ndims = ndims;
    g_fuse.vec = vec ? 1u : 0u;
    g_fuse.nvec = nvec;
    g_fuse.dims[0] = dims[0];
    g_fuse.dims[1] = ndims == 2 ? dims[1] : 1;
    g_fuse.div_inner = make_fastdiv(g_fuse.dims[ndims - 1]);
    g_fuse.nwide = g_fuse.wide_m = g_fuse.wide_nvec = 0;
    g_fuse_elem_bytes = elem_bytes;
}
// The first-space member whose output is, row for row, the left operand of the one-term product `c` over `m` columns
// (the latest that writes any of it), -1 when there is none, -2 when the operand meets such outputs in any other way.
static int own_rows_member(const FuseCmd& c, const ParMember& m, uint32_t wide_m) {
    for (int k = (int)g_fuse.n - 1; k >= 0; --k) {
        if (!m.in[0].overlaps(g_par[k].out)) continue;
        const FuseCmd& e = g_fuse.cmd[k];
        const bool rows = c.op == FUSE_OP_DOT && c.dims[1] == 1 && c.dims[0] == wide_m && c.in[0] == (const void*)e.out && c.is[0][0] == 1 &&
                          e.os[0] == 1 && m.in[0].lo == g_par[k].out.lo && m.in[0].hi == g_par[k].out.hi;
        return rows ? k : -2;
    }
    return -1;
}
// the kernel computes a member's element offsets in 32 bits
static bool offsets_fit(const ParMember& m) {
    const uint64_t limit = 1ull << 33;          // 2^31 elements of four bytes
    return m.out.hi - m.out.lo < limit && m.in[0].hi - m.in[0].lo < limit && m.in[1].hi - m.in[1].lo < limit;
}
// Adds a member to the parallel phase (joining the open chain when it may, closing it and opening a new one otherwise).
static void add_member(const FuseCmd& c, const ParMember& m, uint32_t ndims, const uint32_t* dims, bool vec, size_t nvec, size_t elem_bytes) {
    const uint32_t members = g_fuse.n + g_fuse.nwide;
    bool join = (g_fuse.n > 0 || g_fuse.ntail > 0) && members < (uint32_t)FUSE_MAX_CMDS;
    bool wide = false;
    int own_rows = -1;
    if (join && g_fuse.n > 0) {
        const bool same_form = g_fuse.ndims == ndims && g_fuse.vec == (vec ? 1u : 0u) && g_fuse_elem_bytes == elem_bytes;
        const bool first_space = same_form && g_fuse.nwide == 0 && g_fuse.nvec == nvec && g_fuse.dims[0] == dims[0] && (ndims == 1 || g_fuse.dims[1] == dims[1]);
        if (!first_space) {
            // the wide space: m times the units of a one-dim first space, and staging slots left for m rounds
            const size_t mult = same_form && ndims == 1 && nvec % g_fuse.nvec == 0 ? nvec / g_fuse.nvec : 0;
            wide = mult >= 2 && mult <= (size_t)FUSE_MAX_WIDE && nvec <= 0xFFFFFFFFull / 4 && (g_fuse.nwide == 0 || g_fuse.wide_m == mult) &&
                   g_fuse.n + (g_fuse.nwide + 1) * mult <= (size_t)FUSE_MAX_CMDS;
            if (wide) {
                own_rows = own_rows_member(c, m, (uint32_t)mult);
                wide = own_rows != -2;
            }
            join = wide;
            if (wide && g_fuse.nwide == 0) {
                g_fuse.wide_m = (uint32_t)mult;
                g_fuse.wide_nvec = (uint32_t)nvec;
            }
        }
    }
    if (join) join = clear_of_members(c, m, ndims, wide, own_rows) && clear_of_tail(m, c.nin);
    if (!join) {
        fuse_flush();
        wide = false;
    }
    if (g_fuse.n == 0) open_space(ndims, dims, vec, nvec, elem_bytes);
    const uint32_t at = g_fuse.n + g_fuse.nwide;
    FuseCmd& slot = g_fuse.cmd[at];
    slot = c;
    slot.fwd = 0;
    slot.src = FUSE_SRC_MEMORY | (FUSE_SRC_MEMORY << 8);
    if (c.op != FUSE_OP_DOT) {
        // (FUSE_OP_MSE_BACKWARD included: its two inputs are an elementwise member's)
        // An input that is an earlier member's output (element for element: nothing else was let in) is not in memory yet:
        // the members' stores wait until all of them are done.  It comes from the latest such member's staged output,
        // or straight from registers when that is the member before.  (A wide member only meets wide members so.)
        const int lowest = wide ? (int)g_fuse.n : 0;
        for (uint32_t j = 0; j < c.nin; ++j)
            for (int k = (int)at - 1; k >= lowest; --k) {
                if (!m.in[j].overlaps(g_par[k].out)) continue;
                if ((uint32_t)k + 1 == at) slot.fwd |= 1u << j;
                slot.src = (slot.src & ~(0xFFu << (8 * j))) | ((uint32_t)k << (8 * j));
                break;
            }
    } else if (wide && own_rows >= 0) {
        slot.src = (slot.src & ~0xFFu) | (uint32_t)own_rows;
    }
    // `0 + the member before` (a gradient's first accumulation): that member makes it along with its own output
    const bool after_one_of_its_space = at > (wide ? g_fuse.n : 0u);
    if (after_one_of_its_space && c.op == (uint32_t)IndexOf<OpZeroPlus<float>, EwProgOps>::value && c.nin == 1 && slot.fwd == 1u &&
        !(g_fuse.cmd[at - 1].fwd & FUSE_NEXT_IS_ZERO_PLUS) && (at < 2 || at - 1 == g_fuse.n || !(g_fuse.cmd[at - 2].fwd & FUSE_NEXT_IS_ZERO_PLUS)))
        g_fuse.cmd[at - 1].fwd |= FUSE_NEXT_IS_ZERO_PLUS;
    g_par[at] = m;
    if (wide) ++g_fuse.nwide;
    else ++g_fuse.n;
    ++g_fused_launches;
}

static bool tail_same_thread(const FuseCmd* a, const void* pa, const int64_t* sa, const FuseCmd* b, const void* pb, const int64_t* sb) {
    // thread v owns element v of a stage's own space: two operands are one thread's when the spaces and the mappings agree
    return a && b && a->ndims == b->ndims && a->dims[0] == b->dims[0] && a->dims[1] == b->dims[1] && same_mapping(pa, sa, pb, sb, a->ndims);
}

static bool chain_record_tail(uint32_t kind, uint32_t sub, const void* arg, size_t arg_bytes, const Extent* in, int nin, const Extent& out, size_t outputs) {
    if (!fuse_accepting() || arg_bytes > (size_t)FUSE_TAIL_ARG_BYTES || nin > 2) return false;
    if (g_fuse.ntail >= (uint32_t)FUSE_MAX_TAIL) fuse_flush();
    const uint32_t at = g_fuse.ntail;
    if (at == 0) g_fuse.prefetch = 0;
    TailCmd& t = g_fuse.tail[at];
    std::memset((void*)&t, 0, sizeof(t));
    t.kind = kind;
    t.sub = sub;
    std::memcpy(t.arg, arg, arg_bytes);
    TailStage& st = g_tail[at];
    st.out = out;
    st.nin = nin;
    for (int j = 0; j < 2; ++j) {
        st.in[j] = j < nin ? in[j] : Extent{0, 0};
        st.late[j] = false;
    }
    FuseCmd* c = kind == TAIL_EW ? (FuseCmd*)t.arg : nullptr;
    auto stage_cmd = [&](uint32_t k) { return g_fuse.tail[k].kind == TAIL_EW ? (const FuseCmd*)g_fuse.tail[k].arg : (const FuseCmd*)nullptr; };
    // Stages run in order, but by 256 threads that only meet at barriers.  Work out where each input comes from and
    // which barrier, if any, the stage needs first.
    uint32_t sync = 0;
    if (c) {
        c->src = 0;
        st.mirrored = c->os[c->ndims - 1] == 1 && (c->ndims == 1 || c->os[0] == (int64_t)c->dims[1]);
        for (int j = 0; j < nin; ++j) {
            int writer = -1;                            // the latest earlier stage that writes some of this input
            for (int k = (int)at - 1; k >= 0 && writer < 0; --k)
                if (st.in[j].overlaps(g_tail[k].out)) writer = k;
            uint32_t from = FUSE_SRC_MEMORY;
            if (writer >= 0) {
                const TailStage& w = g_tail[writer];
                const FuseCmd* wc = stage_cmd((uint32_t)writer);
                const bool own = tail_same_thread(c, c->in[j], c->is[j], wc, wc ? wc->out : nullptr, wc ? wc->os : nullptr);
                if (w.mirrored && st.in[j].lo >= w.out.lo && st.in[j].hi <= w.out.hi) {
                    from = (uint32_t)writer;
                    t.moff[j] = (int32_t)((st.in[j].lo - w.out.lo) / sizeof(float));
                    if (own && (uint32_t)writer + 1 == at) t.fwd |= 1u << j;
                    if (!own && (uint32_t)writer >= g_lds_from && sync < 1) sync = 1;
                } else {
                    from = FUSE_SRC_MEMORY_LATE;
                    st.late[j] = true;
                    if (!own && (uint32_t)writer >= g_mem_from) sync = 2;
                }
            }
            c->src |= from << (8 * j);
            if (from == FUSE_SRC_MEMORY) g_fuse.prefetch |= 1u << (2 * at + j);
        }
    } else {
        st.mirrored = outputs <= 256;
        for (int j = 0; j < nin; ++j) {
            st.late[j] = true;
            for (uint32_t k = g_mem_from; k < at; ++k)
                if (st.in[j].overlaps(g_tail[k].out)) sync = 2;
        }
        if (at > 0 && sync < 1) sync = 1;               // the fold's LDS is reused from stage to stage
    }
    // what the stage writes against what unordered earlier stages wrote, or read late, through other threads
    for (uint32_t k = g_mem_from; k < at && sync < 2; ++k) {
        const TailStage& e = g_tail[k];
        const FuseCmd* ec = stage_cmd(k);
        if (st.out.overlaps(e.out) && !tail_same_thread(c, c ? c->out : nullptr, c ? c->os : nullptr, ec, ec ? ec->out : nullptr, ec ? ec->os : nullptr)) sync = 2;
        for (int j = 0; j < e.nin && sync < 2; ++j)
            if (e.late[j] && st.out.overlaps(e.in[j]) &&
                !tail_same_thread(c, c ? c->out : nullptr, c ? c->os : nullptr, ec, ec ? ec->in[j] : nullptr, ec ? ec->is[j] : nullptr)) sync = 2;
    }
    t.sync = sync;
    t.mirrored = st.mirrored ? 1u : 0u;
    if (sync >= 1) g_lds_from = at;
    if (sync == 2) g_mem_from = at;
    ++g_fuse.ntail;
    ++g_fused_launches;
    return true;
}

static bool chain_record(const FuseCmd& c, uint32_t ndims, const uint32_t* dims, bool vec, size_t nvec, size_t elem_bytes) {
    // only once the capture cannot be a whole-capture program any more (that path launches for real)
    if (!fuse_accepting() || ndims < 1 || ndims > 2) return false;
    for (uint32_t d = 0; d < ndims; ++d)
        if (c.os[d] < 0 || c.is[0][d] < 0 || (c.nin > 1 && c.is[1][d] < 0)) return false;
    ParMember m;
    m.out = operand_range(c.out, c.os, ndims, dims, elem_bytes);
    for (uint32_t j = 0; j < 2; ++j) {
        m.in[j] = j < c.nin ? operand_range(c.in[j], c.is[j], ndims, dims, elem_bytes) : Extent{0, 0};
        m.across[j] = false;
    }
    // at most one block's worth of elements, one per thread: a stage of the tail, where a barrier between stages
    // orders everything (any shapes, any overlaps)
    size_t nel = 1;
    for (uint32_t d = 0; d < ndims; ++d) nel *= dims[d];
    if (nel <= 256) {
        FuseCmd t = c;
        t.fwd = 0;
        t.ndims = ndims;
        t.dims[0] = dims[0];
        t.dims[1] = ndims == 2 ? dims[1] : 1;
        t.nel = (uint32_t)nel;
        return chain_record_tail(TAIL_EW, 0, &t, sizeof(t), m.in, (int)c.nin, m.out, nel);
    }
    if (!offsets_fit(m)) return false;
    add_member(c, m, ndims, dims, vec, nvec, elem_bytes);
    return true;
}

static bool chain_record_dot(const FuseCmd& c, size_t outputs, const Extent& x, const Extent& y) {
    if (!fuse_accepting() || outputs <= 256) return false;
    ParMember m;
    m.out = Extent{(uintptr_t)c.out, (uintptr_t)c.out + outputs * sizeof(float)};
    m.in[0] = x;
    m.in[1] = y;
    m.across[0] = m.across[1] = true;
    const bool vec = outputs % 4 == 0 && (uintptr_t)c.out % 16 == 0;
    const uint32_t dims[1] = {(uint32_t)outputs};
    if (!offsets_fit(m)) return false;
    add_member(c, m, 1, dims, vec, vec ? outputs / 4 : outputs, sizeof(float));
    return true;
}

static bool chain_record_mse_backward(const FuseCmd& c, bool vec, size_t nvec, const Extent& grad_loss) {
    if (!fuse_accepting() || c.nel <= 256) return false;
    ParMember m;
    const uint32_t dims[1] = {c.nel};
    m.out = operand_range(c.out, c.os, 1, dims, sizeof(float));
    for (uint32_t j = 0; j < 2; ++j) {
        m.in[j] = operand_range(c.in[j], c.is[j], 1, dims, sizeof(float));
        m.across[j] = false;
    }
    m.extra = grad_loss;
    if (m.extra.overlaps(m.out)) return false;
    if (!offsets_fit(m)) return false;
    add_member(c, m, 1, dims, vec, nvec, sizeof(float));
    return true;
}

// ---- the capture as a resident step program: the launch sites' offers are kept, not launched ---------------------
static bool res_accepting() { return g_res_ok && !g_res_spilling && fuse_accepting(); }

// The capture is not going to be a resident program: what was kept goes to the fused chains in order (which take
// exactly these offers) or is launched, and later offers go there directly.
static void res_spill() {
    if (!g_res_ok) return;
    g_res_ok = false;
    g_res_spilling = true;
    std::vector<ResRecord> recs;
    recs.swap(g_res);
    for (const ResRecord& r : recs)
        if (r.kind != RES_DISCARD) --g_fused_launches;      // counted again by whoever takes them now
    for (ResRecord& r : recs) {
        bool taken = true;
        if (r.kind == RES_DISCARD) continue;
        if (r.kind == RES_EW) taken = chain_record(*(const FuseCmd*)r.arg, r.ndims, r.dims, r.vec, r.units, sizeof(float));
        else if (r.kind == RES_DOT) taken = r.chain_ok && chain_record_dot(*(const FuseCmd*)r.arg, r.outputs, r.in[0], r.in[1]);
        else taken = chain_record_tail(r.tail_kind, r.sub, r.arg, r.arg_bytes, r.in, r.nin, r.out, r.outputs);
        if (!taken) {
            if (r.relaunch) r.relaunch();
            else set_status(ERR_LAUNCH, "a launch kept for a resident step program could be neither fused nor launched");
        }
    }
    g_res_spilling = false;
}

bool fuse_record(const FuseCmd& c, uint32_t ndims, const uint32_t* dims, bool vec, size_t nvec, size_t elem_bytes) {
    if (res_accepting()) {
        bool fits = ndims >= 1 && ndims <= 2 && elem_bytes == sizeof(float) && nvec * (vec ? 4 : 1) <= g_res_elems;
        for (uint32_t d = 0; d < ndims && fits; ++d) fits = c.os[d] >= 0 && c.is[0][d] >= 0 && (c.nin < 2 || c.is[1][d] >= 0);
        if (fits) {
            ResRecord r;
            r.kind = RES_EW;
            r.vec = vec;
            r.ndims = ndims;
            r.dims[0] = dims[0];
            r.dims[1] = ndims == 2 ? dims[1] : 1;
            r.units = nvec;
            std::memset(r.arg, 0, sizeof(r.arg));
            std::memcpy(r.arg, &c, sizeof(c));
            r.arg_bytes = sizeof(c);
            r.nin = (int)c.nin;
            r.out = operand_range(c.out, c.os, ndims, dims, elem_bytes);
            for (uint32_t j = 0; j < c.nin; ++j) r.in[j] = operand_range(c.in[j], c.is[j], ndims, dims, elem_bytes);
            g_res.push_back(std::move(r));
            ++g_fused_launches;
            return true;
        }
        res_spill();
    }
    return chain_record(c, ndims, dims, vec, nvec, elem_bytes);
}

bool fuse_record_dot(const FuseCmd& c, size_t outputs, const Extent& x, const Extent& y, std::function<void()> relaunch, bool chain_ok) {
    if (res_accepting()) {
        if (outputs <= g_res_elems && (x.hi - x.lo) / sizeof(float) <= g_res_elems && ((outputs > 256 && chain_ok) || relaunch)) {
            ResRecord r;
            r.kind = RES_DOT;
            r.vec = outputs % 4 == 0 && (uintptr_t)c.out % 16 == 0;
            r.units = r.vec ? outputs / 4 : outputs;
            r.outputs = outputs;
            std::memset(r.arg, 0, sizeof(r.arg));
            std::memcpy(r.arg, &c, sizeof(c));
            r.arg_bytes = sizeof(c);
            r.nin = 2;
            r.out = Extent{(uintptr_t)c.out, (uintptr_t)c.out + outputs * sizeof(float)};
            r.in[0] = x;
            r.in[1] = y;
            r.relaunch = std::move(relaunch);
            r.chain_ok = chain_ok;
            g_res.push_back(std::move(r));
            ++g_fused_launches;
            return true;
        }
        res_spill();
    }
    return chain_ok && chain_record_dot(c, outputs, x, y);
}

bool fuse_record_tail(uint32_t kind, uint32_t sub, const void* arg, size_t arg_bytes, const Extent* in, int nin, const Extent& out, size_t outputs) {
    if (res_accepting()) {
        bool fits = arg_bytes <= (size_t)FUSE_TAIL_ARG_BYTES && nin >= 1 && nin <= 2 && (kind == TAIL_ROW_REDUCE || kind == TAIL_DOT || kind == TAIL_MSE);
        for (int j = 0; j < nin && fits; ++j) fits = (in[j].hi - in[j].lo) / sizeof(float) <= g_res_elems;
        if (fits) {
            ResRecord r;
            r.kind = kind == TAIL_ROW_REDUCE ? RES_ROW : kind == TAIL_DOT ? RES_TAILDOT : RES_MSE;
            r.tail_kind = kind;
            r.sub = sub;
            r.outputs = outputs;
            std::memset(r.arg, 0, sizeof(r.arg));
            std::memcpy(r.arg, arg, arg_bytes);
            r.arg_bytes = arg_bytes;
            r.nin = nin;
            r.out = out;
            for (int j = 0; j < nin; ++j) r.in[j] = in[j];
            g_res.push_back(std::move(r));
            ++g_fused_launches;
            return true;
        }
        res_spill();
    }
    return chain_record_tail(kind, sub, arg, arg_bytes, in, nin, out, outputs);
}

bool fuse_record_mse_backward(const FuseCmd& c, bool vec, size_t nvec, const Extent& grad_loss) {
    if (res_accepting()) res_spill();      // (a resident step program has no command for it)
    return chain_record_mse_backward(c, vec, nvec, grad_loss);
}

void prog_abandon() {
    if (g_capturing) g_prog_ok = false;
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

static size_t g_scratch_allocs = 0;       // hipMallocs made by scratch() (under g_scratch_mu)

void* scratch(size_t bytes, int slot) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16 || slot < 0 || slot > 2) {
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
    ++g_scratch_allocs;
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
    // Work still queued on the old stream may use the scratch slots and the fixed no-alloc array, which are one per
    // device and which the first call on the new stream may overwrite: drain the old stream.  (Not when it is being
    // captured - by the library or by the caller: nothing is running on it then, and a capture forbids the wait.)
    if ((hipStream_t)s != g_stream && !g_capturing) {
        hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(g_stream, &st) == hipSuccess && st == hipStreamCaptureStatusNone) (void)hipStreamSynchronize(g_stream);
        else (void)hipGetLastError();
    }
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

// hipMallocs the scratch buffers have cost so far (for callers and tests that must see none).
size_t hip_scratch_allocations(void) { std::lock_guard<std::mutex> lk(g_scratch_mu); return g_scratch_allocs; }
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
    int dev = 0;
    (void)hipGetDevice(&dev);
    g_tickets_ready = false;
    if (dev >= 0 && dev < 16) {
        if (!g_tickets[dev]) g_tickets[dev] = fuse_tickets();
        g_tickets_ready = g_tickets[dev] != nullptr;
    }
    e = hipStreamBeginCapture(g_capture_stream, hipStreamCaptureModeThreadLocal);
    if (e != hipSuccess) return (int)e;
    g_saved_stream = g_stream;
    g_stream = g_capture_stream;
    g_capturing = true;
    g_capture_owner = std::this_thread::get_id();
    // a resident step program holds what a whole-capture program holds and more: it takes that one's place
    g_res_ok = g_res_elems > 0 && g_fuse_enabled && g_tickets_ready;
    g_res_spilling = false;
    g_res.clear();
    g_prog_ok = g_prog_enabled && !g_res_ok;
    g_prog_pending = false;
    g_prog_cmds.clear();
    g_fuse.n = 0;
    g_fuse.nwide = g_fuse.wide_m = g_fuse.wide_nvec = 0;
    g_fuse.ntail = 0;
    g_lds_from = g_mem_from = 0;
    g_fused_launches = g_fuse_nodes = 0;
    return 0;
}
int hip_graph_end_capture(void** graph_exec) {
    MXH_API_INT;
    if (!g_capturing || !graph_exec) return (int)hipErrorInvalidValue;
    ResProgram res;
    bool as_res = false;
    if (g_res_ok) {
        as_res = !g_res.empty() && res_build(g_res, res);
        if (as_res) { g_res.clear(); g_res_ok = false; }
        else res_spill();
    }
    fuse_flush();
    hipGraph_t graph = nullptr;
    hipError_t e = hipStreamEndCapture(g_capture_stream, &graph);
    g_stream = g_saved_stream;
    g_capturing = false;
    const bool as_program = g_prog_ok && !g_prog_pending && !g_prog_cmds.empty();
    if (e != hipSuccess) return (int)e;
    GraphExec* ge = new GraphExec();
    if (as_res) {
        // nothing was launched into the capture: replays are one launch of the resident interpreter
        (void)hipGraphDestroy(graph);
        if (!res_upload(res)) { delete ge; return (int)hipErrorOutOfMemory; }
        ge->res = res;
    } else if (as_program) {
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
    if (ge->res.device_cmds) {
        res_launch(ge->res, 1, (void*)s);
        return (int)hipGetLastError();
    }
    if (ge->cmds) {
        prog_launch(ge->cmds, ge->n, (void*)s);
        return (int)hipGetLastError();
    }
    return (int)hipGraphLaunch(ge->graph, s);
}
// `times` replays in a row.  A resident step program makes them in ONE launch: its tensors stay in LDS from the first
// replay to the last, and memory sees the final state (the same bytes as `times` separate replays leave).
int hip_graph_launch_n(void* graph_exec, size_t times) {
    MXH_API_INT;
    if (!graph_exec || !g_capture_stream || g_capturing) return (int)hipErrorInvalidValue;
    GraphExec* ge = (GraphExec*)graph_exec;
    hipStream_t s = g_stream ? g_stream : g_capture_stream;
    if (ge->res.device_cmds) {
        while (times > 0) {
            const uint32_t chunk = (uint32_t)std::min<size_t>(times, 4096);      // bounds one kernel's running time
            res_launch(ge->res, chunk, (void*)s);
            times -= chunk;
        }
        return (int)hipGetLastError();
    }
    for (size_t i = 0; i < times; ++i) {
        hipError_t e = hipSuccess;
        if (ge->cmds) { prog_launch(ge->cmds, ge->n, (void*)s); e = hipGetLastError(); }
        else e = hipGraphLaunch(ge->graph, s);
        if (e != hipSuccess) return (int)e;
    }
    return 0;
}
// Body commands of the resident step program behind `graph_exec` (0: the capture is not one); optionally how many
// operand references it serves from LDS and how many work-group barriers one replay makes.
int hip_graph_is_resident(void* graph_exec, int* lds_operands, int* barriers) {
    if (!graph_exec || !((GraphExec*)graph_exec)->res.device_cmds) return 0;
    const ResProgram& r = ((GraphExec*)graph_exec)->res;
    if (lds_operands) *lds_operands = (int)r.in_lds;
    if (barriers) *barriers = (int)r.barriers;
    return (int)r.n_body;
}
// The largest tensor, in elements, a launch may touch for later captures to stay resident step programs (0: never; at
// most 65536; default 4096); returns the previous setting.
int hip_graph_set_resident(int max_elements) {
    std::lock_guard<std::recursive_mutex> api(g_api_mu);
    const int was = (int)g_res_elems;
    g_res_elems = max_elements <= 0 ? 0 : std::min<size_t>((size_t)max_elements, RES_MAX_ELEMS);
    return was;
}
// The caller no longer needs what [ptr, ptr + bytes) holds (a pooled buffer went back to its pool).  Outside a capture
// nothing happens.  Inside one it lets a resident step program skip the write-back of tensors that nobody will read.
void hip_buffer_discard(void* ptr, size_t bytes) {
    MXH_API;
    if (!g_capturing || !g_res_ok || g_res_spilling || !ptr || bytes == 0) return;
    ResRecord r;
    r.kind = RES_DISCARD;
    r.out = Extent{(uintptr_t)ptr, (uintptr_t)ptr + bytes};
    g_res.push_back(std::move(r));
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
    res_destroy(ge->res);
    delete ge;
    {
        // the last live capture is gone: nothing refers to retired scratch blocks, or to the current ones, any more
        std::lock_guard<std::mutex> lk(g_scratch_mu);
        if (--g_live_captures <= 0) {
            g_live_captures = 0;
            for (void* p : g_retired_scratch) (void)hipFree(p);
            g_retired_scratch.clear();
            for (auto& dev : g_scratch_captured) dev[0] = dev[1] = dev[2] = false;
        }
    }
    return (int)e;
}

}  // extern "C"
