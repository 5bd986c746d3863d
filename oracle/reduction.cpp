// TEST INFRASTRUCTURE ONLY — CPU restatement of crates/maidenx_cpu/src/ops/reduction.rs.
// Metadata layouts:
//   sum/mean/max/min (reduction.rs:28-32): dims[n] | strides[n] | red_len[r] | red_stride[r] | offset
//   sum_to_shape     (reduction.rs:111-114): in_dims[n] | in_strides[n] | out_dims[n] | offset
//   fold             (reduction.rs:298-305): dims[n] | strides[n] | fold_dim, window_dim, fold_size, step, window_size, offset
// The reference accumulates in the storage dtype, one locked `+=` per input element, in
// whatever order rayon schedules.  With one thread this restatement visits input elements
// in ascending logical order (the order a single-threaded rayon pool yields); with several
// threads it replays the per-output-lock scheme and is only used for timing.
#include <atomic>
#include <thread>

#include "common.hpp"

using namespace orc;

namespace {

template <typename T> inline T zero_of() { return T(0); }
template <> inline bf16 zero_of<bf16>() { return bf16::from_f32(0.0f); }
template <> inline f16 zero_of<f16>() { return f16::from_f32(0.0f); }
template <typename T> inline T lowest_of() { return std::numeric_limits<T>::lowest(); }   // f32::MIN
template <> inline bf16 lowest_of<bf16>() { return bf16::from_f32(std::numeric_limits<float>::lowest()); }
template <> inline f16 lowest_of<f16>() { return f16::from_f32(std::numeric_limits<float>::lowest()); }
template <typename T> inline T highest_of() { return std::numeric_limits<T>::max(); }     // f32::MAX
template <> inline bf16 highest_of<bf16>() { return bf16::from_f32(std::numeric_limits<float>::max()); }
template <> inline f16 highest_of<f16>() { return f16::from_f32(std::numeric_limits<float>::max()); }
template <typename T> inline T from_count(size_t n) { return (T)n; }                      // `x as f32`
template <> inline bf16 from_count<bf16>(size_t n) { return bf16::from_f32((float)n); }
template <> inline f16 from_count<f16>(size_t n) { return f16::from_f32((float)n); }

// One lock word + value per output element, like the reference's Vec<Mutex<T>>.
template <typename T> struct Cell {
    std::atomic<uint32_t> lock{0};
    T val;
};
template <typename T, typename F> inline void locked(Cell<T>& c, bool threaded, F f) {
    if (!threaded) { f(c.val); return; }
    uint32_t expect = 0;
    while (!c.lock.compare_exchange_weak(expect, 1, std::memory_order_acquire)) { expect = 0; std::this_thread::yield(); }
    f(c.val);
    c.lock.store(0, std::memory_order_release);
}

// reduction.rs:48-54 / :66-75 — destination of logical input index i.
inline size_t dst_of(size_t i, size_t nred, const size_t* red_l, const size_t* red_s, bool contiguous) {
    size_t dst = i;
    for (size_t nd = 0; nd < nred; ++nd) {
        size_t stride = red_s[nd];
        if (contiguous || stride != 0) {
            size_t pre = dst / stride, post = dst % stride;
            dst = (pre / red_l[nd]) * stride + post;
        } else {
            dst /= red_l[nd];
        }
    }
    return dst;
}

// Shared skeleton of sum_op! (:6-89), mean_op! (:185-272), max_op! (:383-467), min_op! (:469-553).
template <typename T, typename Acc, typename Fin>
void reduce_axis(size_t num_els, size_t num_dims, size_t nred, const size_t* md, const T* inp, T* out, T init,
                 Acc acc, Fin fin) {
    const size_t* dims = md;
    const size_t* strides = md + num_dims;
    const size_t* red_l = md + 2 * num_dims;
    const size_t* red_s = md + 2 * num_dims + nred;
    size_t offset = md[2 * num_dims + 2 * nred];
    const T* in = inp + offset;
    size_t out_size = num_els;
    for (size_t i = 0; i < nred; ++i) out_size /= red_l[i];
    std::vector<Cell<T>> cells(out_size);
    for (auto& c : cells) c.val = init;
    bool threaded = num_threads() > 1;
    bool cont = is_contiguous(num_dims, dims, strides);
    ORC_PAR_FOR
    for (size_t i = 0; i < num_els; ++i) {
        size_t src = cont ? i : get_strided_index(i, num_dims, dims, strides);
        size_t dst = dst_of(i, nred, red_l, red_s, cont);
        T v = in[src];
        locked(cells[dst], threaded, [&](T& o) { acc(o, v); });
    }
    for (size_t i = 0; i < out_size; ++i) out[i] = fin(cells[i].val);
}

// sum_to_shape_op! (:91-183)
template <typename T>
void sum_to_shape(size_t num_els, size_t num_dims, const size_t* md, const T* inp, T* out) {
    const size_t* in_dims = md;
    const size_t* in_strides = md + num_dims;
    const size_t* out_dims = md + 2 * num_dims;
    size_t offset = md[3 * num_dims];
    const T* in = inp + offset;
    size_t out_size = 1;
    for (size_t d = 0; d < num_dims; ++d) out_size *= out_dims[d];
    std::vector<Cell<T>> cells(out_size);
    for (auto& c : cells) c.val = zero_of<T>();
    std::vector<size_t> factor(num_dims);
    for (size_t d = 0; d < num_dims; ++d) factor[d] = in_dims[d] / out_dims[d];
    bool threaded = num_threads() > 1;
    bool cont = is_contiguous(num_dims, in_dims, in_strides);
    ORC_PAR_FOR
    for (size_t i = 0; i < num_els; ++i) {
        size_t coords[16];
        size_t tmp = i;
        for (size_t d = num_dims; d-- > 0;) { coords[d] = tmp % in_dims[d]; tmp /= in_dims[d]; }
        size_t dst = 0;
        for (size_t d = 0; d < num_dims; ++d) dst = dst * out_dims[d] + coords[d] / factor[d];
        size_t src = i;
        if (!cont) {
            // :162-167 — the slice already starts at `offset`, yet the index adds it again, modulo num_els.
            size_t s = 0;
            for (size_t d = 0; d < num_dims; ++d) s += coords[d] * in_strides[d];
            src = (s + offset) % num_els;
        }
        T v = in[src];
        locked(cells[dst], threaded, [&](T& o) { o = add_wrap(o, v); });
    }
    for (size_t i = 0; i < out_size; ++i) out[i] = cells[i].val;
}

// fold_op! (reduction.rs:274-380): the adjoint of unfold.  Input element with coordinates c adds to the
// output at c with the window dim dropped and the fold dim replaced by c[fold_dim]*step + c[window_dim]
// (skipped when that is >= fold_size).  The source index is (sum c*stride) % num_els of the slice that
// starts at `offset` (:336-340), contiguous or not.
// metadata: dims[n] | strides[n] | fold_dim, window_dim, fold_size, step, window_size, offset
template <typename T>
void fold(size_t num_els, size_t nd, const size_t* md, const T* inp, T* out) {
    const size_t* dims = md;
    const size_t* strides = md + nd;
    const size_t fold_dim = md[2 * nd], window_dim = md[2 * nd + 1], fold_size = md[2 * nd + 2], step = md[2 * nd + 3];
    const size_t offset = md[2 * nd + 5];
    const T* in = inp + offset;
    size_t out_size = 1;
    for (size_t d = 0; d < nd; ++d) {
        if (d == window_dim) continue;
        out_size *= d == fold_dim ? fold_size : dims[d];
    }
    std::vector<Cell<T>> cells(out_size);
    for (auto& c : cells) c.val = zero_of<T>();
    bool threaded = num_threads() > 1;
    ORC_PAR_FOR
    for (size_t i = 0; i < num_els; ++i) {
        size_t coords[16] = {0};
        size_t tmp = i;
        for (size_t d = nd; d-- > 0;) { coords[d] = tmp % dims[d]; tmp /= dims[d]; }
        size_t src = 0;
        for (size_t d = 0; d < nd; ++d) src += coords[d] * strides[d];
        src %= num_els;
        size_t pos = coords[fold_dim] * step + coords[window_dim];
        if (pos >= fold_size) continue;
        size_t dst = 0;
        for (size_t d = 0; d < nd; ++d) {
            if (d == window_dim) continue;
            dst = d == fold_dim ? dst * fold_size + pos : dst * dims[d] + coords[d];
        }
        T v = in[src];
        locked(cells[dst], threaded, [&](T& o) { o = add_wrap(o, v); });
    }
    for (size_t i = 0; i < out_size; ++i) out[i] = cells[i].val;
}

}  // namespace

#define ORC_REDUCE_FOR(T, SUF)                                                                                  \
    extern "C" void oracle_sum_##SUF(size_t n, size_t nd, size_t nr, const size_t* md, const T* in, T* out) {   \
        reduce_axis<T>(n, nd, nr, md, in, out, zero_of<T>(), [](T& o, T v) { o = add_wrap(o, v); }, [](T v) { return v; }); \
    }                                                                                                           \
    extern "C" void oracle_mean_##SUF(size_t n, size_t nd, size_t nr, const size_t* md, const T* in, T* out) {  \
        size_t f = 1;                                                                                           \
        for (size_t i = 0; i < nr; ++i) f *= md[2 * nd + i];                                                    \
        T ff = from_count<T>(f); /* :264-268 — divide once, at the end */                                       \
        reduce_axis<T>(n, nd, nr, md, in, out, zero_of<T>(), [](T& o, T v) { o += v; },                         \
                       [ff](T v) { return v / ff; });                                                           \
    }                                                                                                           \
    extern "C" void oracle_max_##SUF(size_t n, size_t nd, size_t nr, const size_t* md, const T* in, T* out) {   \
        reduce_axis<T>(n, nd, nr, md, in, out, lowest_of<T>(), [](T& o, T v) { o = v > o ? v : o; },            \
                       [](T v) { return v; });                                                                  \
    }                                                                                                           \
    extern "C" void oracle_min_##SUF(size_t n, size_t nd, size_t nr, const size_t* md, const T* in, T* out) {   \
        reduce_axis<T>(n, nd, nr, md, in, out, highest_of<T>(), [](T& o, T v) { o = v < o ? v : o; },           \
                       [](T v) { return v; });                                                                  \
    }                                                                                                           \
    extern "C" void oracle_sum_to_shape_##SUF(size_t n, size_t nd, const size_t* md, const T* in, T* out) {     \
        sum_to_shape<T>(n, nd, md, in, out);                                                                    \
    }                                                                                                           \
    extern "C" void oracle_fold_##SUF(size_t n, size_t nd, const size_t* md, const T* in, T* out) {             \
        fold<T>(n, nd, md, in, out);                                                                            \
    }

ORC_REDUCE_FOR(float, f32)
ORC_REDUCE_FOR(double, f64)
ORC_REDUCE_FOR(bf16, bf16)
ORC_REDUCE_FOR(f16, f16)

// the integer dtypes have sum, max, min and sum_to_shape (reduction.rs:559-566, 572-579, 605-612, 618-625); no mean
#define ORC_REDUCE_INT_FOR(T, SUF)                                                                              \
    extern "C" void oracle_sum_##SUF(size_t n, size_t nd, size_t nr, const size_t* md, const T* in, T* out) {   \
        reduce_axis<T>(n, nd, nr, md, in, out, T(0), [](T& o, T v) { o = add_wrap(o, v); }, [](T v) { return v; }); \
    }                                                                                                           \
    extern "C" void oracle_max_##SUF(size_t n, size_t nd, size_t nr, const size_t* md, const T* in, T* out) {   \
        reduce_axis<T>(n, nd, nr, md, in, out, std::numeric_limits<T>::min(), [](T& o, T v) { o = v > o ? v : o; }, \
                       [](T v) { return v; });                                                                  \
    }                                                                                                           \
    extern "C" void oracle_min_##SUF(size_t n, size_t nd, size_t nr, const size_t* md, const T* in, T* out) {   \
        reduce_axis<T>(n, nd, nr, md, in, out, std::numeric_limits<T>::max(), [](T& o, T v) { o = v < o ? v : o; }, \
                       [](T v) { return v; });                                                                  \
    }                                                                                                           \
    extern "C" void oracle_sum_to_shape_##SUF(size_t n, size_t nd, const size_t* md, const T* in, T* out) {     \
        sum_to_shape<T>(n, nd, md, in, out);                                                                    \
    }                                                                                                           \
    extern "C" void oracle_fold_##SUF(size_t n, size_t nd, const size_t* md, const T* in, T* out) {             \
        fold<T>(n, nd, md, in, out);                                                                            \
    }
ORC_REDUCE_INT_FOR(uint8_t, u8)
ORC_REDUCE_INT_FOR(uint16_t, u16)
ORC_REDUCE_INT_FOR(uint32_t, u32)
ORC_REDUCE_INT_FOR(uint64_t, u64)
ORC_REDUCE_INT_FOR(int8_t, i8)
ORC_REDUCE_INT_FOR(int16_t, i16)
ORC_REDUCE_INT_FOR(int32_t, i32)
ORC_REDUCE_INT_FOR(int64_t, i64)
