// TEST INFRASTRUCTURE ONLY — CPU restatement of the host loops of crates/maidenx_tensor/src/ops/indexing.rs
// (index_select :93-124, index_add_ :15-91, index_put_ :182-311, gather :315-363, scatter_add_ :403-461, bincount :463-522) and
// of add_at_index (crates/maidenx_tensor/src/utils/indexing.rs:96-140): indices are read `as_i32`, the
// adds are in the storage dtype, elements are visited in the order the reference's loops visit them.
// A layout is dims[n] | strides[n] | offset.  On an index outside its range the reference returns an
// error from the middle of the loop; this restatement stops there too and reports it through
// oracle_index_error() (the outputs are then only partly written, as in the reference).
#include "common.hpp"

using namespace orc;

namespace {

int g_index_error = 0;

template <typename T> inline T zero_of() { return T(0); }
template <> inline bf16 zero_of<bf16>() { return bf16::from_f32(0.0f); }
template <> inline f16 zero_of<f16>() { return f16::from_f32(0.0f); }

// add_at_index (utils/indexing.rs:121-135): `+` in the storage dtype - wrapping for the integers (the reference's
// release build), `||` for bool.
template <typename T> inline T idx_add(T a, T b) {
    if constexpr (std::is_same<T, bool>::value) return a || b;
    else return add_wrap(a, b);
}

struct Layout {
    size_t nd;
    const size_t *dims, *strides;
    size_t offset;
    Layout(size_t n, const size_t* l) : nd(n), dims(l), strides(l + n), offset(l[2 * n]) {}
    size_t at(const size_t* c) const {
        size_t o = offset;
        for (size_t d = 0; d < nd; ++d) o += c[d] * strides[d];
        return o;
    }
};

// row-major walk over `dims` (index_iter), calling f(coords)
template <typename F> void walk(size_t nd, const size_t* dims, F f) {
    size_t total = 1;
    for (size_t d = 0; d < nd; ++d) total *= dims[d];
    std::vector<size_t> c(nd, 0);
    for (size_t i = 0; i < total; ++i) {
        if (!f(c.data())) return;
        for (size_t d = nd; d-- > 0;) {
            if (++c[d] < dims[d]) break;
            c[d] = 0;
        }
    }
}

template <typename T, typename I>
void index_select(size_t nd, size_t dim, const size_t* in_layout, size_t n_idx, size_t idx_stride, size_t idx_offset, const I* indices,
                  const T* input, T* output) {
    Layout in(nd, in_layout);
    std::vector<size_t> out_dims(in.dims, in.dims + nd), out_str(nd);
    out_dims[dim] = n_idx;
    size_t acc = 1;
    for (size_t d = nd; d-- > 0;) { out_str[d] = acc; acc *= out_dims[d]; }
    std::vector<size_t> slice(out_dims);
    slice[dim] = 1;
    for (size_t i = 0; i < n_idx; ++i) {
        int32_t idx = (int32_t)indices[idx_offset + i * idx_stride];
        if (idx < 0 || idx >= (int32_t)in.dims[dim]) { g_index_error = 1; return; }
        walk(nd, slice.data(), [&](const size_t* c) {
            size_t src = in.offset, dst = 0;
            for (size_t d = 0; d < nd; ++d) {
                src += (d == dim ? (size_t)idx : c[d]) * in.strides[d];
                dst += (d == dim ? i : c[d]) * out_str[d];
            }
            output[dst] = input[src];
            return true;
        });
    }
}

template <typename T, typename I>
void gather(size_t nd, size_t dim, const size_t* in_layout, const size_t* idx_layout, const I* index, const T* input, T* output) {
    Layout in(nd, in_layout), ix(nd, idx_layout);
    size_t o = 0;
    walk(nd, ix.dims, [&](const size_t* c) {
        int32_t v = (int32_t)index[ix.at(c)];
        int32_t size = (int32_t)in.dims[dim];
        int32_t actual = v < 0 ? size + v : v;
        if (actual < 0 || actual >= size) { g_index_error = 1; return false; }
        size_t src = in.offset;
        for (size_t d = 0; d < nd; ++d) src += (d == dim ? (size_t)actual : c[d]) * in.strides[d];
        output[o++] = input[src];
        return true;
    });
}

template <typename T, typename I>
void index_add(size_t nd, size_t dim, const size_t* self_layout, const size_t* src_layout, size_t n_idx, size_t idx_stride,
               size_t idx_offset, const I* indices, const T* src, T* self) {
    Layout sl(nd, self_layout), sr(nd, src_layout);
    std::vector<size_t> slice(sr.dims, sr.dims + nd);
    slice[dim] = 1;
    for (size_t i = 0; i < n_idx; ++i) {
        int32_t idx = (int32_t)indices[idx_offset + i * idx_stride];
        if (idx < 0 || idx >= (int32_t)sl.dims[dim]) { g_index_error = 1; return; }
        walk(nd, slice.data(), [&](const size_t* c) {
            size_t s = sr.offset, d0 = sl.offset;
            for (size_t d = 0; d < nd; ++d) {
                s += (d == dim ? i : c[d]) * sr.strides[d];
                d0 += (d == dim ? (size_t)idx : c[d]) * sl.strides[d];
            }
            self[d0] = idx_add(self[d0], src[s]);
            return true;
        });
    }
}

template <typename T, typename I>
void scatter_add(size_t nd, size_t dim, const size_t* self_layout, const size_t* idx_layout, const size_t* src_layout, const I* index,
                 const T* src, T* self) {
    Layout sl(nd, self_layout), ix(nd, idx_layout), sr(nd, src_layout);
    walk(nd, sr.dims, [&](const size_t* c) {
        int32_t v = (int32_t)index[ix.at(c)];
        int32_t size = (int32_t)sl.dims[dim];
        int32_t actual = v < 0 ? size + v : v;
        if (actual < 0 || actual >= size) { g_index_error = 1; return false; }
        size_t d0 = sl.offset;
        for (size_t d = 0; d < nd; ++d) {
            size_t cd = d == dim ? (size_t)actual : c[d];
            if (cd >= sl.dims[d]) { g_index_error = 1; return false; }      // add_at_index bounds check
            d0 += cd * sl.strides[d];
        }
        self[d0] = idx_add(self[d0], src[sr.at(c)]);
        return true;
    });
}

template <typename I>
void bincount(size_t n, size_t stride, size_t offset, const I* input, size_t out_size, I* output) {
    for (size_t b = 0; b < out_size; ++b) output[b] = 0;
    for (size_t i = 0; i < n; ++i) {
        int32_t v = (int32_t)input[offset + i * stride];
        if (v < 0 || (size_t)v >= out_size) { g_index_error = 1; return; }
        output[v] = (I)((int32_t)output[v] + 1);          // :515-516 — the count is read back `as_i32`
    }
}

template <typename T, typename I>
void bincount_weighted(size_t n, size_t stride, size_t offset, const I* input, size_t w_stride, size_t w_offset, const T* weights,
                       size_t out_size, T* output) {
    for (size_t b = 0; b < out_size; ++b) output[b] = zero_of<T>();
    for (size_t i = 0; i < n; ++i) {
        int32_t v = (int32_t)input[offset + i * stride];
        if (v < 0 || (size_t)v >= out_size) { g_index_error = 1; return; }
        output[v] = output[v] + weights[w_offset + i * w_stride];
    }
}

}  // namespace

// indexing.rs:182-311 with set_index (utils/indexing.rs:67-94).  The checks come in the reference's order; the copy of
// a sub-tensor is its recursion over the source dims (row-major), every dim fixed means one element (0-d source) or
// the element-by-element writes behind indices[0] that only a 1-d self accepts.
template <typename T>
void index_put(size_t self_nd, const size_t* self_layout, size_t n_indices, const size_t* indices, size_t src_nd, const size_t* src_layout,
               const T* src, T* self) {
    Layout sl(self_nd, self_layout), rl(src_nd, src_layout);
    if (n_indices > self_nd) { g_index_error = 1; return; }
    const size_t remaining = self_nd - n_indices;
    if (remaining > 0) {
        if (src_nd != remaining) { g_index_error = 1; return; }
        for (size_t i = 0; i < remaining; ++i)
            if (rl.dims[i] != sl.dims[n_indices + i]) { g_index_error = 1; return; }
        size_t base = 0;
        for (size_t d = 0; d < n_indices; ++d) {
            if (indices[d] >= sl.dims[d]) { g_index_error = 1; return; }
            base += indices[d] * sl.strides[d];
        }
        base += sl.offset;
        walk(src_nd, rl.dims, [&](const size_t* c) {
            size_t dst = base, from = rl.offset;
            for (size_t d = 0; d < src_nd; ++d) { dst += c[d] * sl.strides[n_indices + d]; from += c[d] * rl.strides[d]; }
            self[dst] = src[from];
            return true;
        });
        return;
    }
    auto set_index = [&](const size_t* idx, size_t n, T v) {
        if (n != self_nd) { g_index_error = 1; return false; }
        for (size_t d = 0; d < n; ++d)
            if (idx[d] >= sl.dims[d]) { g_index_error = 1; return false; }
        size_t flat = sl.offset;
        for (size_t d = 0; d < n; ++d) flat += idx[d] * sl.strides[d];
        self[flat] = v;
        return true;
    };
    if (src_nd == 0) { set_index(indices, n_indices, src[rl.offset]); return; }
    size_t src_size = 1, self_size = 1;
    for (size_t i = 0; i < src_nd; ++i) src_size *= rl.dims[i];
    for (size_t i = 0; i < self_nd; ++i) self_size *= sl.dims[i];
    if (src_size == 0) return;
    if (n_indices == 0) { g_index_error = 1; return; }          // indices[0] of an empty slice: a panic in the reference
    const size_t self_dim = indices[0];
    if (self_dim + src_size > self_size) { g_index_error = 1; return; }
    for (size_t i = 0; i < src_size; ++i) {
        size_t one = self_dim + i;
        if (!set_index(&one, 1, src[rl.offset + i * rl.strides[0]])) return;
    }
}

extern "C" int oracle_index_error() { int e = g_index_error; g_index_error = 0; return e; }

#define ORC_INDEX_FOR(T, TS, I, IS)                                                                                                  \
    extern "C" void oracle_index_select_##TS##_##IS(size_t nd, size_t dim, const size_t* in_layout, size_t n_idx, size_t idx_stride, \
                                                    size_t idx_offset, const I* indices, const T* input, T* output) {                \
        index_select<T, I>(nd, dim, in_layout, n_idx, idx_stride, idx_offset, indices, input, output);                               \
    }                                                                                                                                \
    extern "C" void oracle_gather_##TS##_##IS(size_t nd, size_t dim, const size_t* in_layout, const size_t* idx_layout,              \
                                              const I* index, const T* input, T* output) {                                          \
        gather<T, I>(nd, dim, in_layout, idx_layout, index, input, output);                                                          \
    }                                                                                                                                \
    extern "C" void oracle_index_add_##TS##_##IS(size_t nd, size_t dim, const size_t* self_layout, const size_t* src_layout,         \
                                                 size_t n_idx, size_t idx_stride, size_t idx_offset, const I* indices,              \
                                                 const T* src, T* self) {                                                           \
        index_add<T, I>(nd, dim, self_layout, src_layout, n_idx, idx_stride, idx_offset, indices, src, self);                        \
    }                                                                                                                                \
    extern "C" void oracle_scatter_add_##TS##_##IS(size_t nd, size_t dim, const size_t* self_layout, const size_t* idx_layout,       \
                                                   const size_t* src_layout, const I* index, const T* src, T* self) {               \
        scatter_add<T, I>(nd, dim, self_layout, idx_layout, src_layout, index, src, self);                                           \
    }                                                                                                                                \
    extern "C" void oracle_bincount_weighted_##TS##_##IS(size_t n, size_t stride, size_t offset, const I* input, size_t w_stride,    \
                                                         size_t w_offset, const T* weights, size_t out_size, T* output) {           \
        bincount_weighted<T, I>(n, stride, offset, input, w_stride, w_offset, weights, out_size, output);                            \
    }

// bool and the integers (the tensor layer's index ops are dtype-generic through Scalar, indexing.rs:15,93,182,315,403):
// everything but the weighted bincount, whose weights are floats
#define ORC_INDEX_WIDE_FOR(T, TS, I, IS)                                                                                             \
    extern "C" void oracle_index_select_##TS##_##IS(size_t nd, size_t dim, const size_t* in_layout, size_t n_idx, size_t idx_stride, \
                                                    size_t idx_offset, const I* indices, const T* input, T* output) {                \
        index_select<T, I>(nd, dim, in_layout, n_idx, idx_stride, idx_offset, indices, input, output);                               \
    }                                                                                                                                \
    extern "C" void oracle_gather_##TS##_##IS(size_t nd, size_t dim, const size_t* in_layout, const size_t* idx_layout,              \
                                              const I* index, const T* input, T* output) {                                          \
        gather<T, I>(nd, dim, in_layout, idx_layout, index, input, output);                                                          \
    }                                                                                                                                \
    extern "C" void oracle_index_add_##TS##_##IS(size_t nd, size_t dim, const size_t* self_layout, const size_t* src_layout,         \
                                                 size_t n_idx, size_t idx_stride, size_t idx_offset, const I* indices,              \
                                                 const T* src, T* self) {                                                           \
        index_add<T, I>(nd, dim, self_layout, src_layout, n_idx, idx_stride, idx_offset, indices, src, self);                        \
    }                                                                                                                                \
    extern "C" void oracle_scatter_add_##TS##_##IS(size_t nd, size_t dim, const size_t* self_layout, const size_t* idx_layout,       \
                                                   const size_t* src_layout, const I* index, const T* src, T* self) {               \
        scatter_add<T, I>(nd, dim, self_layout, idx_layout, src_layout, index, src, self);                                           \
    }
#define ORC_INDEX_WIDE(T, TS) ORC_INDEX_WIDE_FOR(T, TS, int32_t, i32) ORC_INDEX_WIDE_FOR(T, TS, int64_t, i64) ORC_INDEX_PUT_FOR(T, TS)

ORC_INDEX_FOR(float, f32, int32_t, i32)
ORC_INDEX_FOR(float, f32, int64_t, i64)
ORC_INDEX_FOR(double, f64, int32_t, i32)
ORC_INDEX_FOR(double, f64, int64_t, i64)
ORC_INDEX_FOR(bf16, bf16, int32_t, i32)
ORC_INDEX_FOR(f16, f16, int32_t, i32)
ORC_INDEX_FOR(bf16, bf16, int64_t, i64)
ORC_INDEX_FOR(f16, f16, int64_t, i64)

#define ORC_INDEX_PUT_FOR(T, TS)                                                                                                     \
    extern "C" void oracle_index_put_##TS(size_t self_nd, const size_t* self_layout, size_t n_indices, const size_t* indices,        \
                                          size_t src_nd, const size_t* src_layout, const T* src, T* self) {                         \
        index_put<T>(self_nd, self_layout, n_indices, indices, src_nd, src_layout, src, self);                                       \
    }
ORC_INDEX_PUT_FOR(float, f32)
ORC_INDEX_PUT_FOR(double, f64)
ORC_INDEX_PUT_FOR(bf16, bf16)
ORC_INDEX_PUT_FOR(f16, f16)

extern "C" void oracle_bincount_i32(size_t n, size_t stride, size_t offset, const int32_t* input, size_t out_size, int32_t* output) {
    bincount<int32_t>(n, stride, offset, input, out_size, output);
}
extern "C" void oracle_bincount_i64(size_t n, size_t stride, size_t offset, const int64_t* input, size_t out_size, int64_t* output) {
    bincount<int64_t>(n, stride, offset, input, out_size, output);
}

ORC_INDEX_WIDE(bool, bool)
ORC_INDEX_WIDE(uint8_t, u8)
ORC_INDEX_WIDE(uint16_t, u16)
ORC_INDEX_WIDE(uint32_t, u32)
ORC_INDEX_WIDE(uint64_t, u64)
ORC_INDEX_WIDE(int8_t, i8)
ORC_INDEX_WIDE(int16_t, i16)
ORC_INDEX_WIDE(int32_t, i32)
ORC_INDEX_WIDE(int64_t, i64)
