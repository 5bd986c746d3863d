// TEST INFRASTRUCTURE ONLY — CPU restatement of the host loops of crates/maidenx_tensor/src/ops/indexing.rs
// (index_select :93-124, index_add_ :15-91, gather :315-363, scatter_add_ :403-461, bincount :463-522) and
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
            self[d0] = self[d0] + src[s];
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
        self[d0] = self[d0] + src[sr.at(c)];
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

ORC_INDEX_FOR(float, f32, int32_t, i32)
ORC_INDEX_FOR(float, f32, int64_t, i64)
ORC_INDEX_FOR(double, f64, int32_t, i32)
ORC_INDEX_FOR(double, f64, int64_t, i64)
ORC_INDEX_FOR(bf16, bf16, int32_t, i32)
ORC_INDEX_FOR(f16, f16, int32_t, i32)
ORC_INDEX_FOR(bf16, bf16, int64_t, i64)
ORC_INDEX_FOR(f16, f16, int64_t, i64)

extern "C" void oracle_bincount_i32(size_t n, size_t stride, size_t offset, const int32_t* input, size_t out_size, int32_t* output) {
    bincount<int32_t>(n, stride, offset, input, out_size, output);
}
extern "C" void oracle_bincount_i64(size_t n, size_t stride, size_t offset, const int64_t* input, size_t out_size, int64_t* output) {
    bincount<int64_t>(n, stride, offset, input, out_size, output);
}
