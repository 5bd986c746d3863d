// Strided / broadcast elementwise engine: kernels and the host-side path selection.
//
// Every out-of-place op of the reference writes a contiguous output and reads its operands
// through (dims, strides, offset) metadata; the in-place ops write through the lhs strides.
// The host collapses the iteration space, then picks one of two kernels:
//   ew_nd : each lane owns VEC consecutive elements of the innermost collapsed dim.  The
//           logical→memory index walk (a few multiply-high divisions) is done once per
//           lane-vector, operands with inner stride 1 move as one 128-bit access, operands
//           with inner stride 0 as one scalar load.
//   ew_tr : an operand whose unit stride sits on a non-innermost dim (a transposed view) is
//           read along that dim in 64x64 tiles, turned through LDS, and consumed along the
//           output's innermost dim, so both the read and the write stay coalesced.
#pragma once
#include <cstdlib>
#include <cstring>
#include <type_traits>

#include "mxh.hpp"
#include "ew_registry.hpp"
#include "fuse.hpp"

namespace mxh {

template <class T, int N>
struct alignas(sizeof(T) * N) AVec {
    T v[N];
};

template <int NIN>
struct EwPtrs {
    void* out;
    const void* in[NIN];
};

// Loads and stores of one lane-vector with or without the non-temporal hint (the builtins take plain scalar or vector
// types, so the bytes travel as 32-bit words).
template <int BYTES> struct RawVec { typedef void type; };          // other sizes: plain accesses, no hint
template <> struct RawVec<16> { typedef uint32_t type __attribute__((ext_vector_type(4))); };
template <> struct RawVec<8> { typedef uint32_t type __attribute__((ext_vector_type(2))); };
template <> struct RawVec<4> { typedef uint32_t type; };
template <> struct RawVec<2> { typedef uint16_t type; };
template <> struct RawVec<1> { typedef uint8_t type; };
// (STREAM is a compile-time choice: the compiler merges a hinted and a plain access to one address chosen at run time
// into one plain access.)
template <bool STREAM, class V>
__device__ __forceinline__ V ld_vec(const V* p) {
    using R = typename RawVec<sizeof(V)>::type;
    if constexpr (STREAM && !std::is_void<R>::value) return __builtin_bit_cast(V, __builtin_nontemporal_load((const R*)p));
    else return *p;
}
template <bool STREAM, class V>
__device__ __forceinline__ void st_vec(V* p, const V& v) {
    using R = typename RawVec<sizeof(V)>::type;
    if constexpr (STREAM && !std::is_void<R>::value) __builtin_nontemporal_store(__builtin_bit_cast(R, v), (R*)p);
    else *p = v;
}
// Total bytes of a launch from which the hint is used: beyond the 256 MB last-level cache with room to spare.
constexpr size_t EW_STREAM_BYTES = 192u << 20;

constexpr int EW_BLOCK = 256;
#ifndef MXH_EW_UNR
#define MXH_EW_UNR 4
#endif
constexpr int EW_UNR = MXH_EW_UNR;
constexpr unsigned EW_SMALL_BLOCKS = 256;      // fewer blocks than CUs: see ew_launch

// ---- ew_nd -------------------------------------------------------------------------------
// The body takes its block and thread index as arguments: the kernel passes its own, the interpreter of
// recorded programs virtual ones.
// STREAM: the launch moves more data than the last-level cache holds, so nothing it touches can still be cached when it
// is next needed; whole-vector loads and stores then carry the non-temporal hint, which keeps the stream from displacing
// itself on its way through the caches (contiguous f32 multiply of 268 MB operands: 139 -> 123 us).
// STREAM is a mask: bit 0 the store, bit k + 1 the loads of input k (an input that is broadcast along an outer dim is
// read many times over and keeps plain loads).
template <class Op, int VEC, int UNR = EW_UNR, int STREAM = 0, class Space>
__device__ __forceinline__ void ew_nd_body(const Space& sp, const EwPtrs<Op::NIN>& p, size_t nvec, const Op& op,
                                           unsigned bid, unsigned tid) {
    using In = typename Op::In;
    using Out = typename Op::Out;
    constexpr int NIN = Op::NIN;
    const int last = sp.ndims - 1;
    size_t v0 = (size_t)bid * (EW_BLOCK * UNR) + tid;

    // The operands stay packed, as the words they arrived in, until the arithmetic: a narrow dtype unpacked where it is
    // loaded makes every load wait for its data before the next one is issued (add_u8: one 16-byte load in flight).
    using InVec = AVec<In, VEC>;
    using InRaw = typename RawVec<sizeof(InVec)>::type;
    using Held = std::conditional_t<std::is_void<InRaw>::value, InVec, InRaw>;
    Held vals[UNR][NIN];
    int64_t ooff[UNR];
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
        size_t v = v0 + (size_t)u * EW_BLOCK;
        if (v >= nvec) break;
        int64_t off[NIN + 1];
        if (sp.ndims == 1) {
            size_t i = v * VEC;
#pragma unroll
            for (int k = 0; k <= NIN; ++k) off[k] = (int64_t)i * sp.strides[k][0];
        } else {
            uint32_t r = (uint32_t)v * VEC;
#pragma unroll
            for (int k = 0; k <= NIN; ++k) off[k] = 0;
            for (int d = last; d > 0; --d) {
                uint32_t q, c;
                fd_divmod(r, FastDiv{sp.div[d].d, sp.div[d].mul, sp.div[d].shift}, q, c);   // member by member: `sp` may live in the constant address space
#pragma unroll
                for (int k = 0; k <= NIN; ++k) off[k] += (int64_t)c * sp.strides[k][d];
                r = q;
            }
#pragma unroll
            for (int k = 0; k <= NIN; ++k) off[k] += (int64_t)r * sp.strides[k][0];
        }
        ooff[u] = off[0];
#pragma unroll
        for (int k = 0; k < NIN; ++k) {
            const In* src = (const In*)p.in[k] + off[k + 1];
            if constexpr (VEC == 1) {
                InVec t;
                t.v[0] = src[0];
                vals[u][k] = __builtin_bit_cast(Held, t);
            } else {
                const int64_t s = sp.strides[k + 1][last];
                if (s == 1) {
                    vals[u][k] = k == 0 ? ld_vec<(STREAM & 2) != 0>((const Held*)src) : ld_vec<(STREAM & 4) != 0>((const Held*)src);
                } else if (s == 0) {
                    InVec t;
                    t.v[0] = src[0];
#pragma unroll
                    for (int e = 1; e < VEC; ++e) t.v[e] = t.v[0];
                    vals[u][k] = __builtin_bit_cast(Held, t);
                } else {
                    InVec t;
#pragma unroll
                    for (int e = 0; e < VEC; ++e) t.v[e] = src[(int64_t)e * s];
                    vals[u][k] = __builtin_bit_cast(Held, t);
                }
            }
        }
    }
#pragma unroll
    for (int u = 0; u < UNR; ++u) {
        size_t v = v0 + (size_t)u * EW_BLOCK;
        if (v >= nvec) break;
        AVec<Out, VEC> r;
        InVec x[NIN];
#pragma unroll
        for (int k = 0; k < NIN; ++k) x[k] = __builtin_bit_cast(InVec, vals[u][k]);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            if constexpr (NIN == 1) r.v[e] = op(x[0].v[e]);
            else r.v[e] = op(x[0].v[e], x[1].v[e]);
        }
        Out* dst = (Out*)p.out + ooff[u];
        if constexpr (VEC == 1) {
            dst[0] = r.v[0];
        } else {
            st_vec<(STREAM & 1) != 0>((AVec<Out, VEC>*)dst, r);
        }
    }
}
template <class Op, int VEC, int UNR = EW_UNR, int STREAM = 0>
__global__ __launch_bounds__(EW_BLOCK) void ew_nd_kernel(NdSpace<Op::NIN + 1> sp, EwPtrs<Op::NIN> p, size_t nvec,
                                                         Op op) {
    ew_nd_body<Op, VEC, UNR, STREAM>(sp, p, nvec, op, blockIdx.x, threadIdx.x);
}
// Argument block of one recorded ew_nd launch.
template <class Op>
struct EwProgArgs {
    NdSpace<Op::NIN + 1> sp;
    EwPtrs<Op::NIN> p;
    size_t nvec;
    Op op;
};

// ---- ew_tr -------------------------------------------------------------------------------
constexpr int TR_TILE = 64;

template <int NIN>
struct TrPlan {
    int pdim;              // the dim on which the staged operands have stride 1
    uint32_t staged;       // bit k set: input k goes through LDS
    uint32_t tiles_p, tiles_l;
    FastDiv div_tiles_l, div_tiles_p;
    uint32_t super;        // 8x8 super-tile block order (both tile counts are multiples of 8)
    uint32_t same;         // two inputs, one and the same view (x * x): staged once, read twice from the tile
};

template <class Op>
__global__ __launch_bounds__(EW_BLOCK) void ew_tr_kernel(NdSpace<Op::NIN + 1> sp, EwPtrs<Op::NIN> p, TrPlan<Op::NIN> pl,
                                                         Op op) {
    using In = typename Op::In;
    using Out = typename Op::Out;
    constexpr int NIN = Op::NIN;
    __shared__ In tile[NIN][TR_TILE][TR_TILE + 1];

    const int last = sp.ndims - 1;
    const int pd = pl.pdim;
    // blockIdx.x → (outer, tile_p, tile_l), tile_l fastest
    uint32_t b = blockIdx.x, tl, tp, outer;
    fd_divmod(b, pl.div_tiles_l, b, tl);
    fd_divmod(b, pl.div_tiles_p, outer, tp);
    int64_t base[NIN + 1];
#pragma unroll
    for (int k = 0; k <= NIN; ++k) base[k] = 0;
    {
        uint32_t r = outer;
        for (int d = last - 1; d >= 0; --d) {
            if (d == pd) continue;
            uint32_t q, c;
            fd_divmod(r, sp.div[d], q, c);
#pragma unroll
            for (int k = 0; k <= NIN; ++k) base[k] += (int64_t)c * sp.strides[k][d];
            r = q;
        }
    }
    const uint32_t i0 = tp * TR_TILE, j0 = tl * TR_TILE;   // i along pdim, j along the innermost dim
    const uint32_t np = sp.dims[pd], nl = sp.dims[last];
    const uint32_t tx = threadIdx.x % TR_TILE, ty = threadIdx.x / TR_TILE;
    constexpr int ROWS = EW_BLOCK / TR_TILE;

#pragma unroll
    for (int k = 0; k < NIN; ++k) {
        if (!((pl.staged >> k) & 1u)) continue;
        const In* src = (const In*)p.in[k] + base[k + 1];
        const int64_t sl = sp.strides[k + 1][last];
        for (uint32_t r = ty; r < TR_TILE; r += ROWS) {
            uint32_t i = i0 + tx, j = j0 + r;
            if (i < np && j < nl) tile[k][r][tx] = src[(int64_t)i + (int64_t)j * sl];
        }
    }
    __syncthreads();
    for (uint32_t r = ty; r < TR_TILE; r += ROWS) {
        uint32_t i = i0 + r, j = j0 + tx;
        if (i >= np || j >= nl) continue;
        In x[NIN];
#pragma unroll
        for (int k = 0; k < NIN; ++k) {
            if ((pl.staged >> k) & 1u) x[k] = tile[k][tx][r];
            else
                x[k] = ((const In*)p.in[k])[base[k + 1] + (int64_t)i * sp.strides[k + 1][pd] +
                                            (int64_t)j * sp.strides[k + 1][last]];
        }
        Out o;
        if constexpr (NIN == 1) o = op(x[0]);
        else o = op(x[0], x[1]);
        ((Out*)p.out)[base[0] + (int64_t)i * sp.strides[0][pd] + (int64_t)j * sp.strides[0][last]] = o;
    }
}

// ---- ew_trv: vectorised form of ew_tr ------------------------------------------------------------------
// Tile: TP = 256 bytes of the unit-stride dim p by 64 of the innermost dim.  Phase 1 reads the staged
// operands with 128-bit loads along p (each 16-lane group covers one 256-byte row segment) and
// writes them to LDS as tile[l][p]; phase 2 lets every lane gather VEC values down a column of that
// tile (pitch chosen so that the 64 lanes hit distinct banks), combine them with 128-bit loads of
// the other operands along the innermost dim, and store 128 bits.  Needs every dim and stride
// involved to be a multiple of VEC and 16-byte aligned bases (checked by the host).
template <class T> struct TrvCfg {
    static constexpr int VEC = 16 / sizeof(T);
    static constexpr int TP = 256 / sizeof(T);          // tile extent along p
    static constexpr int TL = 64;                       // tile extent along the innermost dim
    static constexpr int PITCH = sizeof(T) == 4 ? TP + 1 : TP + 2;
};

template <class Op, bool STREAM = false>
__global__ __launch_bounds__(EW_BLOCK) void ew_trv_kernel(NdSpace<Op::NIN + 1> sp, EwPtrs<Op::NIN> p, TrPlan<Op::NIN> pl,
                                                          Op op) {
    using In = typename Op::In;
    using Out = typename Op::Out;
    using Cfg = TrvCfg<In>;
    constexpr int NIN = Op::NIN, VEC = Cfg::VEC, TP = Cfg::TP, TL = Cfg::TL, PITCH = Cfg::PITCH;
    __shared__ __attribute__((aligned(16))) In tile[NIN][TL * PITCH];

    const int last = sp.ndims - 1;
    const int pd = pl.pdim;
    uint32_t b = blockIdx.x, tl, tp, outer;
    fd_divmod(b, pl.div_tiles_l, b, tl);
    fd_divmod(b, pl.div_tiles_p, outer, tp);
    if (pl.super) {
        // Blocks that run at the same time form 8x8 groups of tiles: the reads (rows of the staged
        // operand, one row pitch apart) and the writes (rows of the output, also a pitch apart) then
        // both spread over the memory channels instead of one of them hammering a few.
        constexpr uint32_t S = 8;
        uint32_t lin = tp * pl.tiles_l + tl;
        uint32_t per_row = pl.tiles_l / S;
        uint32_t st = lin / (S * S), in = lin % (S * S);
        tp = (st / per_row) * S + in / S;
        tl = (st % per_row) * S + in % S;
    }
    int64_t base[NIN + 1];
#pragma unroll
    for (int k = 0; k <= NIN; ++k) base[k] = 0;
    {
        uint32_t r = outer;
        for (int d = last - 1; d >= 0; --d) {
            if (d == pd) continue;
            uint32_t q, c;
            fd_divmod(r, sp.div[d], q, c);
#pragma unroll
            for (int k = 0; k <= NIN; ++k) base[k] += (int64_t)c * sp.strides[k][d];
            r = q;
        }
    }
    const uint32_t i0 = tp * TP, j0 = tl * TL;
    const uint32_t np = sp.dims[pd], nl = sp.dims[last];
    const int t = threadIdx.x;

    // phase 1: (TP/VEC) vectors per row of the tile, TL rows
    constexpr int VPR = TP / VEC;                       // 16
    constexpr int N1 = TL * VPR / EW_BLOCK;             // 4 vectors per thread
#pragma unroll
    for (int k = 0; k < NIN; ++k) {
        if (!((pl.staged >> k) & 1u) || (k == 1 && pl.same)) continue;
        const In* src = (const In*)p.in[k] + base[k + 1];
        const int64_t sl = sp.strides[k + 1][last];
        AVec<In, VEC> v[N1];
#pragma unroll
        for (int u = 0; u < N1; ++u) {
            int id = t + u * EW_BLOCK;
            uint32_t j = j0 + id / VPR, i = i0 + (id % VPR) * VEC;
            if (i < np && j < nl) v[u] = ld_vec<STREAM>((const AVec<In, VEC>*)(src + (int64_t)i + (int64_t)j * sl));
        }
#pragma unroll
        for (int u = 0; u < N1; ++u) {
            int id = t + u * EW_BLOCK;
            int jl = id / VPR, il = (id % VPR) * VEC;
            // 32-bit LDS writes: the row pitch is not a multiple of 16 bytes
            const uint32_t* w = (const uint32_t*)&v[u];
            uint32_t* dst = (uint32_t*)(&tile[k][jl * PITCH + il]);
#pragma unroll
            for (int e = 0; e < 4; ++e) dst[e] = w[e];
        }
    }
    __syncthreads();

    // phase 2: rows along p, (TL/VEC) vectors per row
    constexpr int VPL = TL / VEC;
    constexpr int N2 = TP * VPL / EW_BLOCK;             // 4 vectors per thread
#pragma unroll
    for (int u = 0; u < N2; ++u) {
        int id = t + u * EW_BLOCK;
        int il = id / VPL, jl = (id % VPL) * VEC;
        uint32_t i = i0 + il, j = j0 + jl;
        if (i >= np || j >= nl) continue;
        In x[NIN][VEC];
#pragma unroll
        for (int k = 0; k < NIN; ++k) {
            if ((pl.staged >> k) & 1u) {
                if (k == 1 && pl.same) {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) x[1][e] = x[0][e];
                } else {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) x[k][e] = tile[k][(jl + e) * PITCH + il];
                }
            } else {
                const In* src = (const In*)p.in[k] + base[k + 1] + (int64_t)i * sp.strides[k + 1][pd] + (int64_t)j * sp.strides[k + 1][last];
                const int64_t s = sp.strides[k + 1][last];
                if (s == 1) {
                    AVec<In, VEC> tv = ld_vec<STREAM>((const AVec<In, VEC>*)src);
#pragma unroll
                    for (int e = 0; e < VEC; ++e) x[k][e] = tv.v[e];
                } else if (s == 0) {
                    In tv = src[0];
#pragma unroll
                    for (int e = 0; e < VEC; ++e) x[k][e] = tv;
                } else {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) x[k][e] = src[(int64_t)e * s];
                }
            }
        }
        AVec<Out, VEC> o;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            if constexpr (NIN == 1) o.v[e] = op(x[0][e]);
            else o.v[e] = op(x[0][e], x[1][e]);
        }
        st_vec<STREAM>((AVec<Out, VEC>*)((Out*)p.out + base[0] + (int64_t)i * sp.strides[0][pd] + (int64_t)j), o);
    }
}

// While a capture is being recorded: the same launch as a command of a program (functors outside the list
// and large grids are not recorded, which leaves the capture to the HIP graph).
template <class Op>
inline void ew_record(int vec, unsigned blocks, const NdSpace<Op::NIN + 1>& sp, const EwPtrs<Op::NIN>& p, size_t n,
                      const Op& op) {
    constexpr int idx = IndexOf<Op, EwProgOps>::value;
    if constexpr (idx >= 0) {
        static_assert(sizeof(EwProgArgs<Op>) <= PROG_ARG_BYTES, "argument block too large for a command");
        if (!prog_recording() || blocks > PROG_MAX_GRID) return;
        EwProgArgs<Op> a;
        std::memset((void*)&a, 0, sizeof(a));
        a.sp = sp;
        a.p = p;
        a.nvec = n;
        a.op = op;
        prog_record(prog_kid(PF_EW, (uint32_t)(idx * 2 + vec)), blocks, &a, sizeof(a));
    }
}

// While a capture is open: offers an f32 -> f32 launch of ew_nd to the open fused group (true: do not launch).
template <class Op>
inline bool ew_fuse(bool vec, const NdSpace<Op::NIN + 1>& sp, const EwPtrs<Op::NIN>& p, size_t n, const Op& op) {
    constexpr int idx = IndexOf<Op, EwProgOps>::value;
    if constexpr (idx >= 0 && std::is_same<typename Op::In, float>::value && std::is_same<typename Op::Out, float>::value && sizeof(Op) <= 8) {
        // launch-bound sizes only: a large tensor is better off with four vectors per thread
        if (sp.ndims < 1 || sp.ndims > 2 || n >= (size_t)EW_SMALL_BLOCKS * EW_BLOCK * EW_UNR) return false;
        // more than one block: the interpreter of recorded programs has no command for it, so the capture is a HIP graph
        if (prog_recording() && cdiv(n, (size_t)EW_BLOCK * EW_UNR) > PROG_MAX_GRID) prog_abandon();
        FuseCmd c;
        std::memset((void*)&c, 0, sizeof(c));
        c.out = p.out;
        c.op = (uint32_t)idx;
        c.nin = Op::NIN;
        std::memcpy(c.payload, (const void*)&op, sizeof(Op));
        for (int d = 0; d < sp.ndims; ++d) {
            c.os[d] = sp.strides[0][d];
            for (int k = 0; k < Op::NIN; ++k) c.is[k][d] = sp.strides[k + 1][d];
        }
        for (int k = 0; k < Op::NIN; ++k) c.in[k] = p.in[k];
        if (vec && c.os[sp.ndims - 1] != 1) return false;
        return fuse_record(c, (uint32_t)sp.ndims, sp.dims, vec, n, sizeof(float));      // (a tiny member is taken element by element whatever `vec` says)
    }
    return false;
}

// Threshold in force (MXH_STREAM_BYTES in the environment overrides it; 0 switches the hint off).
inline size_t ew_stream_bytes() {
    static const size_t v = [] {
        const char* e = getenv("MXH_STREAM_BYTES");
        return e ? (size_t)strtoull(e, nullptr, 10) : EW_STREAM_BYTES;
    }();
    return v;
}

// ---- ew_trvp: ew_trv for one input, as a persistent grid ---------------------------------------------------------
// The same tiles, worked through by 1024-thread blocks that stay (one vector per thread in either phase): a block writes
// the vector it holds to the tile, and after the barrier fetches the NEXT tile's vector before it gathers, computes and
// stores the current one, so the load's latency passes behind the arithmetic instead of in front of it.  What the
// functor looks like on the device is TrvDeviceOp<Op>: by default the functor itself; lut16.hpp's table functor puts
// its table in LDS in front of the tile (PREFIX bytes).
template <class Op>
struct TrvDeviceOp {
    static constexpr size_t PREFIX = 0;
    Op op;
    __device__ TrvDeviceOp(const Op& o, void*) : op(o) {}
    __device__ typename Op::Out operator()(typename Op::In x) const { return op(x); }
};
constexpr int TRVP_BLOCK = 1024;

template <class Op, bool STREAM>
__global__ __launch_bounds__(TRVP_BLOCK) void ew_trvp_kernel(NdSpace<2> sp, EwPtrs<1> p, TrPlan<1> pl, uint32_t tiles, Op host_op) {
    using T = typename Op::In;
    using Out = typename Op::Out;
    using Cfg = TrvCfg<T>;
    constexpr int VEC = Cfg::VEC, TP = Cfg::TP, TL = Cfg::TL, PITCH = Cfg::PITCH;
    static_assert(Op::NIN == 1 && sizeof(Out) == sizeof(T), "one input, an output of its width");
    static_assert(TL * (TP / VEC) == TRVP_BLOCK && TP * (TL / VEC) == TRVP_BLOCK, "one vector per thread in either phase");
    extern __shared__ __attribute__((aligned(16))) unsigned char trvp_smem[];
    T* tile = (T*)(trvp_smem + TrvDeviceOp<Op>::PREFIX);
    const TrvDeviceOp<Op> op(host_op, trvp_smem);

    const int last = sp.ndims - 1, pd = pl.pdim, t = threadIdx.x;
    const uint32_t np = sp.dims[pd], nl = sp.dims[last];
    const int64_t sl = sp.strides[1][last], so = sp.strides[0][pd];
    const int jl1 = t / (TP / VEC), il1 = (t % (TP / VEC)) * VEC;      // phase 1: a vector of row jl1 of the tile
    const int il2 = t / (TL / VEC), jl2 = (t % (TL / VEC)) * VEC;      // phase 2: a vector of output row il2
    struct Tile { int64_t in, out; uint32_t i0, j0; };
    auto locate = [&](uint32_t b) {
        uint32_t tl, tp, outer;
        fd_divmod(b, pl.div_tiles_l, b, tl);
        fd_divmod(b, pl.div_tiles_p, outer, tp);
        if (pl.super) {            // the 8x8 groups of ew_trv_kernel
            constexpr uint32_t S = 8;
            const uint32_t lin = tp * pl.tiles_l + tl, per_row = pl.tiles_l / S, st = lin / (S * S), in = lin % (S * S);
            tp = (st / per_row) * S + in / S;
            tl = (st % per_row) * S + in % S;
        }
        Tile r;
        r.in = 0; r.out = 0;
        for (int d = last - 1; d >= 0; --d) {
            if (d == pd) continue;
            uint32_t q, c;
            fd_divmod(outer, sp.div[d], q, c);
            r.out += (int64_t)c * sp.strides[0][d];
            r.in += (int64_t)c * sp.strides[1][d];
            outer = q;
        }
        r.i0 = tp * TP; r.j0 = tl * TL;
        return r;
    };
    AVec<T, VEC> v;
    bool have = false;
    auto fetch = [&](const Tile& w) {
        const uint32_t i = w.i0 + il1, j = w.j0 + jl1;
        have = i < np && j < nl;
        if (have) v = ld_vec<STREAM>((const AVec<T, VEC>*)((const T*)p.in[0] + w.in + (int64_t)i + (int64_t)j * sl));
    };
    uint32_t b = blockIdx.x;
    Tile cur;
    if (b < tiles) { cur = locate(b); fetch(cur); }
    __syncthreads();               // whatever TrvDeviceOp put into LDS is in place
    for (; b < tiles; b += gridDim.x) {
        if (have) {
            // 32-bit LDS writes: the row pitch is not a multiple of 16 bytes
            const uint32_t* w = (const uint32_t*)&v;
            uint32_t* dst = (uint32_t*)(tile + jl1 * PITCH + il1);
#pragma unroll
            for (int e = 0; e < 4; ++e) dst[e] = w[e];
        }
        __syncthreads();
        const Tile now = cur;
        if (b + gridDim.x < tiles) { cur = locate(b + gridDim.x); fetch(cur); }
        const uint32_t i = now.i0 + il2, j = now.j0 + jl2;
        if (i < np && j < nl) {
            AVec<Out, VEC> o;
#pragma unroll
            for (int e = 0; e < VEC; ++e) o.v[e] = op(tile[(jl2 + e) * PITCH + il2]);
            st_vec<STREAM>((AVec<Out, VEC>*)((Out*)p.out + now.out + (int64_t)i * so + (int64_t)j), o);
        }
        __syncthreads();           // the tile is free again
    }
}

// compute units of a device (0: unknown)
inline int device_cus(int dev) {
    static int cus[16] = {0};
    if (dev < 0 || dev >= 16) return 0;
    if (!cus[dev]) {
        hipDeviceProp_t prop;
        if (hipGetDeviceProperties(&prop, dev) != hipSuccess) { (void)hipGetLastError(); return 0; }
        cus[dev] = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    }
    return cus[dev];
}

// Host: the persistent form when it applies (false: the caller launches ew_trv_kernel).
template <class Op>
inline bool ew_trvp_launch(const NdSpace<Op::NIN + 1>& sp, const EwPtrs<Op::NIN>& p, const TrPlan<Op::NIN>& pl, size_t tiles, bool streams, const Op& op) {
    // Only for functors that keep something in LDS.  For the others it was measured on [8192,8192] and left: 4 to 6 %
    // faster for the cheapest f32 functors (neg 111 -> 104 us), no change for 16-bit ones, 4 to 5 % slower for exp, tanh
    // and gelu in f32, whose arithmetic the barriers of a 1024-thread block then hold up.
    if constexpr (Op::NIN == 1 && TrvDeviceOp<Op>::PREFIX != 0 && sizeof(typename Op::Out) == sizeof(typename Op::In) &&
                  (sizeof(typename Op::In) == 2 || sizeof(typename Op::In) == 4)) {
        using Cfg = TrvCfg<typename Op::In>;
        constexpr size_t PREFIX = TrvDeviceOp<Op>::PREFIX;
        constexpr size_t LDS = PREFIX + (size_t)Cfg::TL * Cfg::PITCH * sizeof(typename Op::In);
        constexpr int PER_CU = 1;                              // blocks a CU holds next to PREFIX bytes
        static bool attr_set[16][2] = {{false}};
        int dev = 0;
        if (pl.staged != 1u || tiles >= (1ull << 32) || hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 16) return false;
        const int cus = device_cus(dev);
        if (!cus || tiles < 64) return false;                  // (the other kernel reads the functor's table from memory)
        if (LDS > 48 * 1024 && !attr_set[dev][streams]) {
            hipError_t e = streams ? hipFuncSetAttribute((const void*)ew_trvp_kernel<Op, true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS)
                                   : hipFuncSetAttribute((const void*)ew_trvp_kernel<Op, false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS);
            if (e != hipSuccess) { (void)hipGetLastError(); return false; }
            attr_set[dev][streams] = true;
        }
        const unsigned grid = (unsigned)std::min<size_t>((size_t)cus * PER_CU, tiles);
        if (streams) hipLaunchKernelGGL((ew_trvp_kernel<Op, true>), dim3(grid), dim3(TRVP_BLOCK), LDS, stream(), sp, p, pl, (uint32_t)tiles, op);
        else hipLaunchKernelGGL((ew_trvp_kernel<Op, false>), dim3(grid), dim3(TRVP_BLOCK), LDS, stream(), sp, p, pl, (uint32_t)tiles, op);
        MXH_LAUNCH_CHECK("ew_trvp");
        return true;
    } else {
        return false;
    }
}

// ---- host-side selection -------------------------------------------------------------------
// in_strides[k] / out_strides are in elements, pointers already include the operand offsets.
template <class Op>
void ew_launch(size_t num_els, size_t num_dims, const size_t* dims, const size_t* out_strides,
               const size_t* const* in_strides, void* out, const void* const* in, Op op) {
    using In = typename Op::In;
    using Out = typename Op::Out;
    constexpr int NIN = Op::NIN;
    if (num_els == 0) return;
    NdSpace<NIN + 1> sp;
    const size_t* strides[NIN + 1];
    strides[0] = out_strides;
    for (int k = 0; k < NIN; ++k) strides[k + 1] = in_strides[k];
    if (!collapse<NIN + 1>(num_dims, dims, strides, sp)) {
        set_status(ERR_UNSUPPORTED, "elementwise: collapsed rank above 8");
        return;
    }
    if (sp.ndims > 1 && num_els >= (1ull << 31)) {
        set_status(ERR_TOO_LARGE, "elementwise: strided op with 2^31 or more elements");
        return;
    }
    EwPtrs<NIN> p;
    p.out = out;
    for (int k = 0; k < NIN; ++k) p.in[k] = in[k];
    const bool streams = ew_stream_bytes() != 0 && num_els * (sizeof(Out) + NIN * sizeof(In)) >= ew_stream_bytes();
    const int last = sp.ndims - 1;

    // transposed-view path?
    if (sp.ndims >= 2 && sp.strides[0][last] == 1 && sp.dims[last] >= 32) {
        int pd = -1;
        uint32_t staged = 0;
        for (int k = 0; k < NIN; ++k) {
            int64_t sl = sp.strides[k + 1][last];
            if (sl == 0 || sl == 1) continue;
            for (int d = 0; d < last; ++d)
                if (sp.strides[k + 1][d] == 1 && sp.dims[d] >= 32 && (pd < 0 || pd == d)) {
                    pd = d;
                    staged |= 1u << k;
                    break;
                }
        }
        if (pd >= 0) {
            TrPlan<NIN> pl;
            pl.pdim = pd;
            pl.staged = staged;
            // vector form: every access of 16 bytes must be aligned and never straddle a tile edge
            constexpr int TV = TrvCfg<In>::VEC;
            // (a narrower output - the bool of a comparison - leaves as vectors of the same element count)
            bool trv = sizeof(Out) <= sizeof(In) && sp.dims[pd] % TV == 0 && sp.dims[last] % TV == 0 &&
                       (uintptr_t)out % 16 == 0;
            for (int d = 0; d < last && trv; ++d) trv = sp.strides[0][d] % TV == 0;
            for (int k = 0; k < NIN && trv; ++k) {
                bool st = (staged >> k) & 1u;
                int64_t sl = sp.strides[k + 1][last];
                if (!st && sl != 1) continue;                      // scalar reads: no constraint
                trv = (uintptr_t)in[k] % 16 == 0;
                for (int d = 0; d <= last && trv; ++d) {
                    if (st && d == pd) continue;
                    if (!st && d == last) continue;
                    trv = sp.strides[k + 1][d] % TV == 0;
                }
            }
            pl.super = 0;
            pl.same = 0;
            if constexpr (NIN == 2) {
                bool same = staged == 3u && in[0] == in[1];
                for (int d = 0; d <= last && same; ++d) same = sp.strides[1][d] == sp.strides[2][d];
                pl.same = same ? 1u : 0u;
            }
            if constexpr (sizeof(In) == 2 || sizeof(In) == 4) if (trv) {      // (the vector tiles are laid out for 16- and 32-bit elements)
                pl.tiles_p = cdiv(sp.dims[pd], TrvCfg<In>::TP);
                pl.tiles_l = cdiv(sp.dims[last], TrvCfg<In>::TL);
                pl.super = (pl.tiles_p % 8 == 0 && pl.tiles_l % 8 == 0) ? 1u : 0u;
                pl.div_tiles_l = make_fastdiv(pl.tiles_l);
                pl.div_tiles_p = make_fastdiv(pl.tiles_p);
                size_t outer = 1;
                for (int d = 0; d < last; ++d)
                    if (d != pd) outer *= sp.dims[d];
                size_t blocks = outer * pl.tiles_p * pl.tiles_l;
                if (ew_trvp_launch<Op>(sp, p, pl, blocks, streams, op)) return;
                if (streams) hipLaunchKernelGGL((ew_trv_kernel<Op, true>), dim3((unsigned)blocks), dim3(EW_BLOCK), 0, stream(), sp, p, pl, op);
                else hipLaunchKernelGGL((ew_trv_kernel<Op, false>), dim3((unsigned)blocks), dim3(EW_BLOCK), 0, stream(), sp, p, pl, op);
                MXH_LAUNCH_CHECK("ew_trv");
                return;
            }
            pl.tiles_p = cdiv(sp.dims[pd], TR_TILE);
            pl.tiles_l = cdiv(sp.dims[last], TR_TILE);
            pl.div_tiles_l = make_fastdiv(pl.tiles_l);
            pl.div_tiles_p = make_fastdiv(pl.tiles_p);
            size_t outer = 1;
            for (int d = 0; d < last; ++d)
                if (d != pd) outer *= sp.dims[d];
            size_t blocks = outer * pl.tiles_p * pl.tiles_l;
            hipLaunchKernelGGL(ew_tr_kernel<Op>, dim3((unsigned)blocks), dim3(EW_BLOCK), 0, stream(), sp, p, pl, op);
            MXH_LAUNCH_CHECK("ew_tr");
            return;
        }
    }

    // vector width: 16 bytes of the wider of In/Out
    constexpr int VEC = 16 / (sizeof(In) > sizeof(Out) ? sizeof(In) : sizeof(Out));
    bool vec_ok = sp.strides[0][last] == 1 && sp.dims[last] % VEC == 0;
    auto aligned = [&](const void* ptr, size_t esz, int k) {
        if (((uintptr_t)ptr) % (esz * VEC) != 0) return false;
        for (int d = 0; d < last; ++d)
            if (sp.strides[k][d] % VEC != 0) return false;
        return true;
    };
    if (vec_ok) vec_ok = aligned(out, sizeof(Out), 0);
    for (int k = 0; k < NIN && vec_ok; ++k)
        if (sp.strides[k + 1][last] == 1) vec_ok = aligned(in[k], sizeof(In), k + 1);
    // A launch that cannot give every CU a block is latency bound: one vector per thread then spreads it over
    // four times as many blocks (a 10000-element powf: 3 blocks of 16 elements per thread otherwise).
    if (vec_ok) {
        size_t nvec = num_els / VEC;
        unsigned blocks = cdiv(nvec, EW_BLOCK * EW_UNR);
        if (ew_fuse<Op>(true, sp, p, nvec, op)) return;
        ew_record<Op>(1, blocks, sp, p, nvec, op);
        if (blocks < EW_SMALL_BLOCKS)
            hipLaunchKernelGGL((ew_nd_kernel<Op, VEC, 1>), dim3(cdiv(nvec, EW_BLOCK)), dim3(EW_BLOCK), 0, stream(), sp, p, nvec, op);
        else if (streams) {
            // an input with a zero stride on some dim is re-read along that dim: plain loads for it
            bool bc[2] = {false, false};
            for (int k = 0; k < NIN; ++k)
                for (int d = 0; d <= last; ++d) bc[k] |= sp.strides[k + 1][d] == 0;
            if constexpr (NIN == 2) {
                if (bc[0] && bc[1]) hipLaunchKernelGGL((ew_nd_kernel<Op, VEC, EW_UNR, 1>), dim3(blocks), dim3(EW_BLOCK), 0, stream(), sp, p, nvec, op);
                else if (bc[1]) hipLaunchKernelGGL((ew_nd_kernel<Op, VEC, EW_UNR, 3>), dim3(blocks), dim3(EW_BLOCK), 0, stream(), sp, p, nvec, op);
                else if (bc[0]) hipLaunchKernelGGL((ew_nd_kernel<Op, VEC, EW_UNR, 5>), dim3(blocks), dim3(EW_BLOCK), 0, stream(), sp, p, nvec, op);
                else hipLaunchKernelGGL((ew_nd_kernel<Op, VEC, EW_UNR, 7>), dim3(blocks), dim3(EW_BLOCK), 0, stream(), sp, p, nvec, op);
            } else {
                if (bc[0]) hipLaunchKernelGGL((ew_nd_kernel<Op, VEC, EW_UNR, 1>), dim3(blocks), dim3(EW_BLOCK), 0, stream(), sp, p, nvec, op);
                else hipLaunchKernelGGL((ew_nd_kernel<Op, VEC, EW_UNR, 3>), dim3(blocks), dim3(EW_BLOCK), 0, stream(), sp, p, nvec, op);
            }
        } else
            hipLaunchKernelGGL((ew_nd_kernel<Op, VEC>), dim3(blocks), dim3(EW_BLOCK), 0, stream(), sp, p, nvec, op);
    } else {
        unsigned blocks = cdiv(num_els, EW_BLOCK * EW_UNR);
        if (ew_fuse<Op>(false, sp, p, num_els, op)) return;
        ew_record<Op>(0, blocks, sp, p, num_els, op);
        if (blocks < EW_SMALL_BLOCKS)
            hipLaunchKernelGGL((ew_nd_kernel<Op, 1, 1>), dim3(cdiv(num_els, EW_BLOCK)), dim3(EW_BLOCK), 0, stream(), sp, p, num_els, op);
        else
            hipLaunchKernelGGL((ew_nd_kernel<Op, 1>), dim3(blocks), dim3(EW_BLOCK), 0, stream(), sp, p, num_els, op);
    }
    MXH_LAUNCH_CHECK("ew_nd");
}

// ---- metadata adapters (layouts of the reference's tensor layer) ---------------------------
// binary / in-place: dims[n] | lhs_strides[n] | rhs_strides[n] | lhs_offset | rhs_offset
template <class Op>
void ew_binary(size_t num_els, size_t num_dims, const size_t* md, const void* lhs, const void* rhs, void* out, Op op,
               bool inplace) {
    using In = typename Op::In;
    if (num_els == 0) return;
    if ((!inplace && !out) || !lhs || !rhs) { set_status(ERR_INVALID, "binary: null buffer"); return; }
    size_t one = num_els, unit = 1;
    const size_t *dims, *ls, *rs;
    size_t lo = 0, ro = 0;
    size_t cont[64];
    if (md == nullptr) { dims = &one; ls = rs = &unit; num_dims = 1; }
    else {
        if (num_dims > 64) { set_status(ERR_INVALID, "binary: rank above 64"); return; }
        dims = md; ls = md + num_dims; rs = md + 2 * num_dims;
        lo = md[3 * num_dims]; ro = md[3 * num_dims + 1];
    }
    const In* l = (const In*)lhs + lo;
    const In* r = (const In*)rhs + ro;
    const size_t* ins[2] = {ls, rs};
    const void* inp[2] = {l, r};
    if (inplace) {
        ew_launch<Op>(num_els, num_dims, dims, ls, ins, (void*)l, inp, op);
    } else {
        contiguous_strides(num_dims, dims, cont);
        ew_launch<Op>(num_els, num_dims, dims, cont, ins, out, inp, op);
    }
}

// unary (+constant): dims[n] | strides[n] | offset ; a null input means "in place on out".
template <class Op>
void ew_unary(size_t num_els, size_t num_dims, const size_t* md, const void* input, void* out, Op op) {
    using In = typename Op::In;
    if (num_els == 0) return;
    if (!out) { set_status(ERR_INVALID, "unary: null output"); return; }
    size_t one = num_els, unit = 1;
    const size_t *dims, *st;
    size_t off = 0;
    size_t cont[64];
    if (md == nullptr) { dims = &one; st = &unit; num_dims = 1; }
    else {
        if (num_dims > 64) { set_status(ERR_INVALID, "unary: rank above 64"); return; }
        dims = md; st = md + num_dims; off = md[2 * num_dims];
    }
    contiguous_strides(num_dims, dims, cont);
    const void* src;
    const size_t* ins[1];
    if (input == nullptr) { src = out; ins[0] = cont; }
    else { src = (const In*)input + off; ins[0] = st; }
    const void* inp[1] = {src};
    ew_launch<Op>(num_els, num_dims, dims, cont, ins, out, inp, op);
}

}  // namespace mxh
