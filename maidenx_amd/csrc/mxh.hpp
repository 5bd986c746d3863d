// Shared host/device helpers of the maidenx_hip backend (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

#include "program.hpp"

namespace mxh {

// ---- status codes returned by hip_get_last_status() ------------------------------------
enum Status : int {
    OK = 0,
    ERR_INVALID = 1,       // bad argument (null pointer, rank above MAXD, malformed metadata)
    ERR_OOM = 2,           // allocation failed (the reference maps code 2 to OutOfMemory)
    ERR_TOO_LARGE = 3,     // a strided op with 2^31 or more logical elements
    ERR_LAUNCH = 4,        // the HIP runtime reported an error (see hip_status_string)
    ERR_UNSUPPORTED = 5,
};

constexpr int MAXD = 8;        // collapsed rank supported by the strided kernels
constexpr int WAVE = 64;

void set_status(int code, const char* what, int hip_err = 0);
hipStream_t stream();

// Every extern "C" entry point holds the library's one lock from its first line to its return, so host threads may call
// in concurrently (the reference's buffers are Send + Sync, crates/maidenx_core/src/buffer/mod.rs:36): calls are
// serialised, and everything a call queues lands on the stream in one piece.  The lock is recursive (entry points call
// each other).  While a graph capture is open, the stream, the fusion group and the command list belong to the thread
// that opened it: a call from another thread is refused (`ok` false, status ERR_INVALID) instead of being recorded into
// that thread's graph.
struct ApiGuard {
    bool ok;
    ApiGuard();
    ~ApiGuard();
    ApiGuard(const ApiGuard&) = delete;
    ApiGuard& operator=(const ApiGuard&) = delete;
};
#define MXH_API                    \
    ::mxh::ApiGuard api_guard__;   \
    if (!api_guard__.ok) return
#define MXH_API_INT                \
    ::mxh::ApiGuard api_guard__;   \
    if (!api_guard__.ok) return (int)hipErrorStreamCaptureWrongThread
// Device scratch owned by the library (three independent slots per device), grown on demand and
// reused by every call; safe because all work of the backend is ordered on one stream.
void* scratch(size_t bytes, int slot = 0);
// runtime.hip: a graph capture is being recorded (nothing may be allocated or grown)
bool capture_open();
// The 65536-entry tables of exp for bf16 / f16 on the current device (lut16.hpp; defined next to the unary entry points);
// null while they cannot be built (a graph capture is open and the table does not exist yet).
const uint16_t* lut16_exp_bf16();
const uint16_t* lut16_exp_f16();
// One int per device that kernels set to 1 when they meet an index outside its range; taking the
// pointer marks it as possibly set, and hip_get_last_status() then reads and clears it.
int* index_flag();

#define MXH_HIP(expr)                                                                 \
    do {                                                                              \
        hipError_t e__ = (expr);                                                      \
        if (e__ != hipSuccess) ::mxh::set_status(::mxh::ERR_LAUNCH, #expr, (int)e__); \
    } while (0)
#define MXH_LAUNCH_CHECK(name)            \
    do {                                  \
        MXH_HIP(hipGetLastError());       \
        ::mxh::prog_launch_seen();        \
    } while (0)

// ---- bf16 storage type -----------------------------------------------------------------
// Same bits as the `half` crate's bf16 the reference stores: upper half of a binary32,
// round-to-nearest-even from f32, NaN kept NaN by forcing the quiet bit.
struct bf16_t {
    uint16_t bits;
};
__host__ __device__ inline float bf2f(bf16_t h) {
    union { uint32_t u; float f; } c;
    c.u = (uint32_t)h.bits << 16;
    return c.f;
}
__host__ __device__ inline bf16_t f2bf(float f) {
#if defined(__HIP_DEVICE_COMPILE__)
    // gfx950 converts in hardware (v_cvt_pk_bf16_f32): round to nearest even, NaN stays a quiet NaN
    bf16_t h;
    h.bits = __builtin_bit_cast(uint16_t, (__bf16)f);
    return h;
#endif
    union { uint32_t u; float f; } c;
    c.f = f;
    uint32_t x = c.u;
    bf16_t r;
    if ((x & 0x7FFFFFFFu) > 0x7F800000u) { r.bits = (uint16_t)((x >> 16) | 0x0040u); return r; }
    // RNE: add 0x7FFF + lsb of the kept part (equivalent to the round-bit/sticky test)
    x += 0x7FFFu + ((x >> 16) & 1u);
    r.bits = (uint16_t)(x >> 16);
    return r;
}

// ---- f16 storage type -------------------------------------------------------------------
// IEEE binary16 as the `half` crate's f16 stores it; conversions are the hardware's
// (round to nearest even; the crate's software path gives the same bits).
struct f16_t {
    uint16_t bits;
};
__host__ __device__ inline float h2f(f16_t h) { return (float)__builtin_bit_cast(_Float16, h.bits); }
__host__ __device__ inline f16_t f2h(float f) {
    f16_t r;
    r.bits = __builtin_bit_cast(uint16_t, (_Float16)f);
    return r;
}

// ---- division by an invariant 32-bit integer (numerators below 2^31) ---------------------
struct FastDiv {
    uint32_t d, mul, shift;
};
inline FastDiv make_fastdiv(uint32_t d) {
    FastDiv f;
    f.d = d;
    if (d <= 1) { f.mul = 0; f.shift = 0; return f; }
    uint32_t s = 0;
    while ((1ull << s) < d) ++s;
    f.shift = s;
    f.mul = (uint32_t)((((1ull << 32) * ((1ull << s) - d)) / d) + 1);
    return f;
}
__device__ inline uint32_t fd_div(uint32_t n, const FastDiv& f) { return (__umulhi(n, f.mul) + n) >> f.shift; }
__device__ inline void fd_divmod(uint32_t n, const FastDiv& f, uint32_t& q, uint32_t& r) {
    q = fd_div(n, f);
    r = n - q * f.d;
}

// ---- collapsed N-d iteration space shared by NOPS operands -------------------------------
// Operand 0 is the output.  Strides are in elements.  After collapse() no dim has size 1 and
// no two neighbouring dims can be merged for every operand at once.
template <int NOPS>
struct NdSpace {
    int ndims;
    uint32_t dims[MAXD];
    FastDiv div[MAXD];
    int64_t strides[NOPS][MAXD];
};

// Host: drop size-1 dims and merge neighbours d, d+1 when stride[d] == stride[d+1] * dim[d+1]
// holds for every operand.  Returns false when the collapsed rank exceeds MAXD.
template <int NOPS>
inline bool collapse(size_t num_dims, const size_t* dims, const size_t* const* strides, NdSpace<NOPS>& out) {
    uint64_t cd[64];
    int64_t cs[NOPS][64];
    int n = 0;
    if (num_dims > 64) return false;
    for (size_t d = 0; d < num_dims; ++d) {
        if (dims[d] == 1) continue;
        bool merge = n > 0;
        if (merge)
            for (int k = 0; k < NOPS; ++k)
                if ((uint64_t)cs[k][n - 1] != (uint64_t)strides[k][d] * dims[d]) { merge = false; break; }
        if (merge) {
            cd[n - 1] *= dims[d];
            for (int k = 0; k < NOPS; ++k) cs[k][n - 1] = (int64_t)strides[k][d];
        } else {
            cd[n] = dims[d];
            for (int k = 0; k < NOPS; ++k) cs[k][n] = (int64_t)strides[k][d];
            ++n;
        }
    }
    if (n == 0) {   // scalar or all-ones shape: one element
        cd[0] = 1;
        for (int k = 0; k < NOPS; ++k) cs[k][0] = 1;
        n = 1;
    }
    if (n > MAXD) return false;
    out.ndims = n;
    for (int d = 0; d < MAXD; ++d) {
        out.dims[d] = d < n ? (uint32_t)cd[d] : 1;
        out.div[d] = make_fastdiv(out.dims[d]);
        for (int k = 0; k < NOPS; ++k) out.strides[k][d] = d < n ? cs[k][d] : 0;
    }
    return true;
}

// Contiguous (row-major) strides of `dims`, as the output of every out-of-place op has.
inline void contiguous_strides(size_t num_dims, const size_t* dims, size_t* strides) {
    size_t acc = 1;
    for (size_t d = num_dims; d-- > 0;) { strides[d] = acc; acc *= dims[d]; }
}

// The reference's contiguity test (size-1 dims ignored).
inline bool ref_is_contiguous(size_t num_dims, const size_t* dims, const size_t* strides) {
    size_t acc = 1;
    for (size_t d = num_dims; d-- > 0;) {
        if (dims[d] > 1 && acc != strides[d]) return false;
        acc *= dims[d];
    }
    return true;
}

inline unsigned cdiv(size_t a, size_t b) { return (unsigned)((a + b - 1) / b); }

}  // namespace mxh
