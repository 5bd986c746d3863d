// TEST INFRASTRUCTURE ONLY — CPU restatement of crates/maidenx_cpu/src/ops/padding.rs: constant,
// reflection and replication padding, forward and backward.
// Metadata layout (padding.rs:31-35):
//   in_dims[n] | in_strides[n] | in_offset | out_dims[n] | (pad_before, pad_after)[n]
#include "common.hpp"

using namespace orc;

namespace {

template <typename T> inline T zero_of() { return T(0); }
template <> inline bf16 zero_of<bf16>() { return bf16::from_f32(0.0f); }
template <> inline f16 zero_of<f16>() { return f16::from_f32(0.0f); }

struct PadMeta {
    const size_t *in_dims, *in_strides, *out_dims, *pads;
    size_t in_off;
    bool cont;
};
inline PadMeta parse(size_t nd, const size_t* md) {
    PadMeta p;
    p.in_dims = md; p.in_strides = md + nd; p.in_off = md[2 * nd];
    p.out_dims = md + 2 * nd + 1; p.pads = md + 3 * nd + 1;
    p.cont = is_contiguous(nd, p.in_dims, p.in_strides);
    return p;
}

// padding.rs:57-98 / :381-418 — output index → input index or "outside".
inline bool map_index(const PadMeta& p, size_t nd, size_t i, size_t* in_idx) {
    size_t out_c[16];
    long in_c[16];
    size_t tmp = i;
    for (size_t d = nd; d-- > 0;) { out_c[d] = tmp % p.out_dims[d]; tmp /= p.out_dims[d]; }
    for (size_t d = 0; d < nd; ++d) {
        in_c[d] = (long)out_c[d] - (long)p.pads[2 * d];
        if (in_c[d] < 0 || in_c[d] >= (long)p.in_dims[d]) return false;
    }
    size_t idx = 0;
    if (p.cont) {
        size_t stride = 1;
        for (size_t d = nd; d-- > 0;) { idx += (size_t)in_c[d] * stride; stride *= p.in_dims[d]; }
    } else {
        for (size_t d = 0; d < nd; ++d) idx += (size_t)in_c[d] * p.in_strides[d];
    }
    *in_idx = idx;
    return true;
}

// pad_with_constant_op! (padding.rs:7-113)
template <typename T>
void pad_const(size_t n_in, size_t n_out, size_t nd, const size_t* md, const T* inp, T* out, T pad_value) {
    (void)n_in;
    PadMeta p = parse(nd, md);
    const T* in = inp + p.in_off;
    ORC_PAR_FOR
    for (size_t i = 0; i < n_out; ++i) {
        size_t src;
        out[i] = map_index(p, nd, i, &src) ? in[src] : pad_value;
    }
}

// pad_with_constant_backward_op! (padding.rs:327-436).  Every input position is hit by
// exactly one output position, so the per-chunk buffers the reference sums through reduce
// to `0 + 0 + … + g`: the value itself, with −0 turned into +0 (:358,420,427).
template <typename T>
void pad_const_backward(size_t n_in, size_t n_out, size_t nd, const size_t* md, const T* grad_out, T* grad_in) {
    PadMeta p = parse(nd, md);
    std::vector<T> g(n_in, zero_of<T>());
    for (size_t i = 0; i < n_out; ++i) {
        size_t dst;
        if (map_index(p, nd, i, &dst)) g[dst] = add_wrap(g[dst], grad_out[i]);
    }
    for (size_t i = 0; i < n_in; ++i) { grad_in[p.in_off + i] = add_wrap(zero_of<T>(), g[i]); }
}

// Reflection (padding.rs:177-195, :497-516) and replication (:289-295, :617-622): output coordinate →
// input coordinate, one dim at a time.  Reflection mirrors at 0 and at dim-1 until the position is
// inside; a dim of size 1 with padding never gets there in the reference (it loops for ever), so the
// restatement requires dim > 1 wherever a dim is padded.
enum class Edge { Reflect, Replicate };

inline long edge_pos(Edge mode, long pos, long dim) {
    if (mode == Edge::Replicate) return pos < 0 ? 0 : (pos > dim - 1 ? dim - 1 : pos);
    if (pos < 0) pos = -pos;
    else if (pos >= dim) pos = 2 * dim - pos - 2;
    while (pos < 0 || pos >= dim) {
        if (pos < 0) pos = -pos;
        else pos = 2 * dim - pos - 2;
    }
    return pos;
}

inline size_t edge_index(const PadMeta& p, Edge mode, size_t nd, size_t i) {
    size_t out_c[16];
    size_t in_c[16];
    size_t tmp = i;
    for (size_t d = nd; d-- > 0;) { out_c[d] = tmp % p.out_dims[d]; tmp /= p.out_dims[d]; }
    for (size_t d = 0; d < nd; ++d) in_c[d] = (size_t)edge_pos(mode, (long)out_c[d] - (long)p.pads[2 * d], (long)p.in_dims[d]);
    size_t idx = 0;
    if (p.cont) {
        size_t stride = 1;
        for (size_t d = nd; d-- > 0;) { idx += in_c[d] * stride; stride *= p.in_dims[d]; }
    } else {
        for (size_t d = 0; d < nd; ++d) idx += in_c[d] * p.in_strides[d];
    }
    return idx;
}

// pad_with_reflection_op! (padding.rs:115-219), pad_with_replication_op! (:221-325)
template <typename T>
void pad_edge(Edge mode, size_t n_in, size_t n_out, size_t nd, const size_t* md, const T* inp, T* out) {
    (void)n_in;
    PadMeta p = parse(nd, md);
    const T* in = inp + p.in_off;
    ORC_PAR_FOR
    for (size_t i = 0; i < n_out; ++i) out[i] = in[edge_index(p, mode, nd, i)];
}

// pad_with_reflection_backward_op! (:438-555), pad_with_replication_backward_op! (:557-665): every output
// gradient is added to the input position it was read from.  The reference sums chunk-local buffers in
// scheduling order; with one chunk the order is ascending output index, which is what this does.
template <typename T>
void pad_edge_backward(Edge mode, size_t n_in, size_t n_out, size_t nd, const size_t* md, const T* grad_out, T* grad_in) {
    PadMeta p = parse(nd, md);
    std::vector<T> g(n_in, zero_of<T>());
    for (size_t i = 0; i < n_out; ++i) { T& c = g[edge_index(p, mode, nd, i)]; c = add_wrap(c, grad_out[i]); }
    for (size_t i = 0; i < n_in; ++i) { grad_in[p.in_off + i] = add_wrap(zero_of<T>(), g[i]); }
}

}  // namespace

#define ORC_PAD_FOR(T, SUF)                                                                                  \
    extern "C" void oracle_pad_with_constant_##SUF(size_t n_in, size_t n_out, size_t nd, const size_t* md,   \
                                                   const T* in, T* out, T pad_value) {                       \
        pad_const<T>(n_in, n_out, nd, md, in, out, pad_value);                                               \
    }                                                                                                        \
    extern "C" void oracle_pad_with_constant_backward_##SUF(size_t n_in, size_t n_out, size_t nd,            \
                                                            const size_t* md, const T* go, T* gi) {          \
        pad_const_backward<T>(n_in, n_out, nd, md, go, gi);                                                  \
    }                                                                                                        \
    extern "C" void oracle_pad_with_reflection_##SUF(size_t n_in, size_t n_out, size_t nd, const size_t* md, \
                                                     const T* in, T* out) {                                  \
        pad_edge<T>(Edge::Reflect, n_in, n_out, nd, md, in, out);                                            \
    }                                                                                                        \
    extern "C" void oracle_pad_with_replication_##SUF(size_t n_in, size_t n_out, size_t nd, const size_t* md,\
                                                      const T* in, T* out) {                                 \
        pad_edge<T>(Edge::Replicate, n_in, n_out, nd, md, in, out);                                          \
    }                                                                                                        \
    extern "C" void oracle_pad_with_reflection_backward_##SUF(size_t n_in, size_t n_out, size_t nd,          \
                                                              const size_t* md, const T* go, T* gi) {        \
        pad_edge_backward<T>(Edge::Reflect, n_in, n_out, nd, md, go, gi);                                    \
    }                                                                                                        \
    extern "C" void oracle_pad_with_replication_backward_##SUF(size_t n_in, size_t n_out, size_t nd,         \
                                                               const size_t* md, const T* go, T* gi) {       \
        pad_edge_backward<T>(Edge::Replicate, n_in, n_out, nd, md, go, gi);                                  \
    }

ORC_PAD_FOR(float, f32)
ORC_PAD_FOR(double, f64)
ORC_PAD_FOR(bf16, bf16)
ORC_PAD_FOR(f16, f16)
// the integers (padding.rs:670-677, 683-690, 696-703, 710-717, 723-730, 736-743): copies forward, wrapping sums backward
ORC_PAD_FOR(uint8_t, u8)
ORC_PAD_FOR(uint16_t, u16)
ORC_PAD_FOR(uint32_t, u32)
ORC_PAD_FOR(uint64_t, u64)
ORC_PAD_FOR(int8_t, i8)
ORC_PAD_FOR(int16_t, i16)
ORC_PAD_FOR(int32_t, i32)
ORC_PAD_FOR(int64_t, i64)
