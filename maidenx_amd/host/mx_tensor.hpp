// Host layer above the backend C ABI: the tensor, autograd and nn calls of MaidenX, restated in C++ so
// that whole training steps (Linear + MSELoss + SGD, Conv2d) can be driven through the backend kernels
// exactly as the reference's tensor layer drives `maidenx_core::be::*`.
//
// Every operation builds the same metadata array and issues the same backend calls, in the same order,
// as the reference function it names:
//   crates/maidenx_tensor/src/lib.rs            Tensor, TensorNode, backward, accumulate_grad, zero_grad
//   crates/maidenx_tensor/src/ops/binary.rs     add sub mul div add_ sub_
//   crates/maidenx_tensor/src/ops/unary.rs      neg square relu tanh gelu exp *_scalar pow gt_scalar
//   crates/maidenx_tensor/src/ops/reduction.rs  sum sum_all sum_to_shape mean mean_all
//   crates/maidenx_tensor/src/ops/matmul.rs     matmul and its backward
//   crates/maidenx_tensor/src/ops/transform.rs  view squeeze unsqueeze transpose broadcast reshape
//   crates/maidenx_core/src/layout.rs           Layout
//   crates/maidenx_nn/src/{layers/linear.rs,layers/conv.rs,losses/mse.rs,optimizers/sgd.rs}
//
// The code is a template over a Backend: a struct of static functions (memory, the f32 kernels, and the
// few helpers the reference runs on the host: fill, strided copy, bool -> f32 cast, scalar broadcast).
// Float tensors are f32 or bf16 (bool results of comparisons); Conv2d is f32 only.
//
// Deliberate differences from the reference, none visible in results:
//   * buffers come from a size-bucketed pool instead of one device allocation per tensor;
//   * `with_buffer_mut`'s copy-on-write of a shared buffer (lib.rs:166-180) is not reproduced: in-place
//     ops write the buffer they are given;
//   * contiguous(), zeros/ones, bool -> f32 and the broadcast of a 0-d tensor run on the device when the
//     backend offers a kernel for them (the reference goes through host memory);
//   * the reference zero-fills the outputs of sum, sum_to_shape and matmul_backward from the host before the
//     kernel overwrites them, and zero-fills every gradient when it is created: the first is skipped (the kernels
//     write every output element), the second is deferred until the zeros are needed (see GradCell).
#pragma once
#include <cmath>
#include <cstdint>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <map>
#include <memory>
#include <set>
#include <stdexcept>
#include <string>
#include <unordered_set>
#include <vector>

namespace mxt {

// ---- errors: the variants of crates/maidenx_core/src/error.rs this layer can raise -------------------
enum class ErrKind { None = 0, InvalidShape, ShapeMismatch, DimensionOutOfBounds, IncompatibleShape, InvalidOperation,
                     InvalidArgument, UnsupportedDType, OutOfMemory, Backend };
struct Error : std::runtime_error {
    ErrKind kind;
    Error(ErrKind k, const std::string& m) : std::runtime_error(m), kind(k) {}
};

using Shape = std::vector<size_t>;
inline size_t shape_size(const Shape& s) { size_t n = 1; for (size_t d : s) n *= d; return n; }
inline std::string shape_str(const Shape& s) {
    std::string r = "[";
    for (size_t i = 0; i < s.size(); ++i) r += (i ? ", " : "") + std::to_string(s[i]);
    return r + "]";
}

// ---- crates/maidenx_core/src/layout.rs ------------------------------------------------------------
struct Layout {
    Shape shape, strides;
    size_t offset = 0;
    static Shape compute_strides(const Shape& shape) {               // layout.rs:337-349
        Shape st(shape.size(), 1);
        for (size_t i = shape.size(); i-- > 1;) st[i - 1] = st[i] * shape[i];
        return st;
    }
    static Layout from_shape(const Shape& s) { return Layout{s, compute_strides(s), 0}; }
    size_t ndim() const { return shape.size(); }
    size_t size() const { return shape_size(shape); }
    bool is_contiguous() const {                                      // layout.rs:60-74 (size-1 dims count)
        size_t expected = 1;
        for (size_t i = ndim(); i-- > 0;) {
            if (strides[i] != expected) return false;
            expected *= shape[i];
        }
        return true;
    }
    void view(const Shape& ns) {                                      // layout.rs:76-97
        if (size() != shape_size(ns))
            throw Error(ErrKind::IncompatibleShape, "Cannot reshape layout of size " + std::to_string(size()) + " to size " +
                                                        std::to_string(shape_size(ns)));
        if (!is_contiguous())
            throw Error(ErrKind::InvalidOperation, "Cannot view a non-contiguous tensor. Use .contiguous() before .view()");
        shape = ns;
        strides = compute_strides(ns);
    }
    void transpose(size_t d0, size_t d1) {                            // layout.rs:99-113
        if (d0 >= ndim() || d1 >= ndim()) throw Error(ErrKind::DimensionOutOfBounds, "transpose: dimension out of bounds");
        std::swap(shape[d0], shape[d1]);
        std::swap(strides[d0], strides[d1]);
    }
    Layout broadcast_to(const Shape& target) const {                  // layout.rs:252-296
        if (shape.size() > target.size())
            throw Error(ErrKind::InvalidArgument, "Cannot broadcast tensor of rank " + std::to_string(shape.size()) + " to rank " +
                                                      std::to_string(target.size()));
        size_t diff = target.size() - shape.size();
        Layout r{target, Shape(target.size(), 0), offset};
        for (size_t i = 0; i < target.size(); ++i) {
            size_t src = i < diff ? 1 : shape[i - diff];
            if (src == target[i]) r.strides[i] = i < diff ? 0 : strides[i - diff];
            else if (src == 1) r.strides[i] = 0;
            else throw Error(ErrKind::InvalidShape, "Cannot broadcast shape " + shape_str(shape) + " to shape " + shape_str(target) +
                                                        " at dimension " + std::to_string(i));
        }
        return r;
    }
};

enum class DType { F32, BF16, BOOL };
inline size_t dtype_size(DType d) { return d == DType::F32 ? 4 : d == DType::BF16 ? 2 : 1; }
inline bool is_float(DType d) { return d != DType::BOOL; }
// crates/maidenx_tensor/src/utils/promotion.rs:16-33, for the dtypes that exist here
inline DType promoted(DType a, DType b) { return a == b ? a : (a == DType::F32 || b == DType::F32) ? DType::F32 : DType::BF16; }

// bf16 as the `half` crate stores it: the high half of an f32, round to nearest even, NaN kept quiet
inline uint16_t f32_to_bf16(float f) {
    uint32_t x;
    std::memcpy(&x, &f, 4);
    if ((x & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((x >> 16) | 0x0040u);
    return (uint16_t)((x + 0x7FFFu + ((x >> 16) & 1u)) >> 16);
}
inline float bf16_to_f32(uint16_t b) {
    uint32_t x = (uint32_t)b << 16;
    float f;
    std::memcpy(&f, &x, 4);
    return f;
}
template <class E> inline E scalar_as(float c);
template <> inline float scalar_as<float>(float c) { return c; }
template <> inline uint16_t scalar_as<uint16_t>(float c) { return f32_to_bf16(c); }     // be/ops/unary.rs:312: constant.as_<dtype>()

// element type tags for the two float dtypes: float, and uint16_t holding bf16 bits
template <class E> struct Tag { using type = E; };
template <class F>
void by_dtype(DType dt, const char* what, F&& f) {
    if (dt == DType::F32) f(Tag<float>{});
    else if (dt == DType::BF16) f(Tag<uint16_t>{});
    else throw Error(ErrKind::UnsupportedDType, std::string(what) + ": needs a float tensor");
}
enum BinOp { ADD, SUB, MUL, DIV };
enum InplaceOp { ADD_INPLACE, SUB_INPLACE };
enum UnOp { NEG, SQUARE, RELU, TANH, GELU, EXP, SQRT };
enum UncOp { ADD_SCALAR, MUL_SCALAR, DIV_SCALAR, POW };
enum RedOp { SUM, MEAN };
// a float scalar with an integer value keeps the tensor's dtype, any other promotes it to f32
// (ops/unary.rs:796-800, 872-876; crates/maidenx_core/src/scalar.rs:115-133)
inline bool integer_valued(float c) { return c == std::trunc(c); }

// ---- buffers: pooled backend memory ------------------------------------------------------------------
// All kernels of a backend run in call order on one stream, so a block handed back to the pool can be
// given to the next tensor at once: whatever still reads it was queued earlier.
template <class B>
struct Pool {
    // Free blocks per bucket, lowest address first: which block a request gets then depends only on the set of
    // free blocks, not on the order they came back in, so a repeated call sequence settles into repeating addresses.
    std::map<size_t, std::set<void*>> free_blocks;
    size_t cached = 0, live = 0, device_allocs = 0;
    std::vector<void*>* trace = nullptr;        // when set, every block handed out is appended (see train loop)
    static constexpr size_t kMaxCached = size_t(64) << 30;
    static size_t bucket(size_t bytes) {
        if (bytes <= 256) return 256;
        if (bytes <= (size_t(1) << 20)) { size_t b = 256; while (b < bytes) b <<= 1; return b; }
        const size_t g = size_t(2) << 20;
        return (bytes + g - 1) / g * g;
    }
    void* get(size_t bytes, size_t& cap) {
        cap = bucket(bytes);
        auto it = free_blocks.find(cap);
        if (it != free_blocks.end() && !it->second.empty()) {
            void* p = *it->second.begin();
            it->second.erase(it->second.begin());
            cached -= cap;
            live += cap;
            if (trace) trace->push_back(p);
            return p;
        }
        void* p = B::alloc(cap);
        if (!p) {                       // give cached blocks back and try once more
            trim();
            p = B::alloc(cap);
            if (!p) throw Error(ErrKind::OutOfMemory, "out of memory");
        }
        ++device_allocs;
        live += cap;
        if (trace) trace->push_back(p);
        return p;
    }
    void put(void* p, size_t cap) {
        live -= cap;
        B::discard(p, cap);             // nobody needs the contents any more (a recorded step may then keep them out of memory)
        if (cached + cap > kMaxCached) { B::sync(); B::free(p); return; }
        free_blocks[cap].insert(p);
        cached += cap;
    }
    void trim() {
        B::sync();
        for (auto& kv : free_blocks)
            for (void* p : kv.second) B::free(p);
        free_blocks.clear();
        cached = 0;
    }
    static Pool& instance() { static Pool* p = new Pool(); return *p; }   // never destroyed: outlives every tensor
};

template <class B>
struct Storage {
    void* ptr = nullptr;
    size_t cap = 0, len = 0;        // len in elements
    explicit Storage(size_t elems, DType dt) : len(elems) { ptr = Pool<B>::instance().get(std::max<size_t>(1, elems) * dtype_size(dt), cap); }
    ~Storage() { Pool<B>::instance().put(ptr, cap); }
    Storage(const Storage&) = delete;
    Storage& operator=(const Storage&) = delete;
};

template <class B> struct Node;
template <class B> struct Tensor;
// The gradient of a tensor.  The reference allocates and zero-fills it in with_grad() and zero_grad()
// (wt.rs:100, lib.rs:262) and the first accumulate_grad adds into those zeros.  Here the zeros stay virtual until
// someone needs them: the first accumulation of a contiguous gradient of the same shape writes 0 + g straight into
// a fresh buffer (the identity sum_to_shape kernel, the same bits as zeros then add_inplace), anything else
// materialises the zeros first.
template <class B> struct GradCell {
    std::shared_ptr<Tensor<B>> g;      // null while the gradient is still all zeros
    Shape shape;
    DType dtype = DType::F32;
};

// Count of backend kernel calls (what `be::*` would dispatch), for reporting.
inline size_t& backend_calls() { static size_t n = 0; return n; }
// Conv2d backward: make only the rows of grad_cols that col2im reads (see Conv2d); false = the whole product.
inline bool& conv_skip_unread_grad_cols() { static bool on = true; return on; }
// sum_all() of a contiguous f32 tensor, and the bias gradient of Conv2d (sums over W, H and the batch), as one reduction
// (true) or dim by dim as the reference does (false).
inline bool& sum_all_in_one_pass() { static bool on = true; return on; }
// Conv2d on a backend that has the product with the gathered column matrix (the matrix is never stored): 0 = store
// the matrix with im2col and multiply that, as the reference does; 1 = gather when no backward is recorded (the
// forward alone is faster gathered, a training step is faster with the one stored matrix serving both products);
// 2 = gather in forward and backward (no buffer of B*oh*ow x C*kh*kw elements lives between the two).
inline int& conv_gathered_products() { static int mode = 1; return mode; }
// What backward() leaves out without changing a bit of any gradient (false: do all of it, as the reference does): the
// gradient of a binary op's or a matmul's operand that does not require one (the reference computes it and drops it,
// lib.rs:93-111),
// x.pow(1) in the backward of pow(2) (x itself), the zero-filled buffer that the first gradient of a tensor is added
// into when that gradient is a broadcast view (0 + g is written straight away, as for a contiguous gradient), and that
// `0 + g` altogether when g is a fresh sum_to_shape result (sums that started from +0: it becomes the gradient as it is).
inline bool& autograd_shortcuts() { static bool on = true; return on; }
// Nesting depth of backward() on this thread.  Inside it tensors are temporaries of the walk - nobody writes into them in
// place - so a result that would be a bit-for-bit copy of its input (`0 + x` of sums that started from +0) may be that
// input, or a view of it.
inline int& backward_depth() { static thread_local int depth = 0; return depth; }
struct BackwardScope {
    BackwardScope() { ++backward_depth(); }
    ~BackwardScope() { --backward_depth(); }
};
// MSELoss and SGD::step as one backend call each where the backend has the fused kernels (the same element functions in
// the same order: every gradient and parameter is the same bytes; the loss is summed in a tree of its own, within the f32
// tolerance of a reduction).  false: the op sequences of the reference.
inline bool& fused_nn_kernels() { static bool on = true; return on; }
// Count of whole-buffer dtype conversions (with_dtype: a host loop in the reference, a kernel here).
inline size_t& cast_calls() { static size_t n = 0; return n; }

// ---- Tensor (crates/maidenx_tensor/src/lib.rs:21-58): shared data, own metadata, optional node ------
template <class B>
struct Tensor {
    std::shared_ptr<Storage<B>> buf;
    std::shared_ptr<GradCell<B>> grad_cell;      // shared by clones, like Arc<Mutex<Tensor>>
    Layout layout;
    DType dtype = DType::F32;
    bool requires_grad = false;
    // This tensor's elements are sums that started from +0 (what sum_to_shape, sum and matmul write: +0 plus anything is
    // never -0), so `0 + x` would copy it bit for bit.  Kept by reshaping views of a tensor that records no gradient.
    bool sums_from_zero = false;
    // The seed of backward() - ones_like(loss), lib.rs:293-301 - not yet written anywhere: a tensor without a buffer that
    // only a backward closure which asked for it (Node::takes_unit_seed) ever sees.
    bool unit_seed = false;
    std::shared_ptr<Node<B>> node;

    using T = Tensor<B>;
    using BackwardFn = std::function<std::vector<T>(const std::vector<T>&, const T&)>;

    // -- accessors --
    const Shape& shape() const { return layout.shape; }
    const Shape& strides() const { return layout.strides; }
    size_t offset() const { return layout.offset; }
    size_t size() const { return layout.size(); }
    size_t ndim() const { return layout.ndim(); }
    bool is_contiguous() const { return layout.is_contiguous(); }
    const float* f32() const { return (const float*)buf->ptr; }
    float* f32() { return (float*)buf->ptr; }
    template <class E> E* p() const { return (E*)buf->ptr; }
    template <class E> using K = typename B::template K<E>;

    // -- creation (creation.rs) --
    static T empty(const Shape& shape, DType dt = DType::F32) {                     // creation.rs:115-131
        T t;
        t.layout = Layout::from_shape(shape);
        t.dtype = dt;
        t.buf = std::make_shared<Storage<B>>(t.layout.size(), dt);
        return t;
    }
    static T fill(const Shape& shape, float v, DType dt = DType::F32) {             // creation.rs:253-305
        T t = empty(shape, dt);
        by_dtype(dt, "fill", [&](auto tag) {
            using E = typename decltype(tag)::type;
            K<E>::fill(t.size(), t.template p<E>(), scalar_as<E>(v));
        });
        return t;
    }
    static T zeros(const Shape& shape, DType dt = DType::F32) { return fill(shape, 0.0f, dt); }   // creation.rs:144-176
    static T ones(const Shape& shape, DType dt = DType::F32) { return fill(shape, 1.0f, dt); }
    static T zeros_like(const T& s) { return zeros(s.shape(), s.dtype); }
    static T ones_like(const T& s) { return ones(s.shape(), s.dtype); }
    static T from_host(const float* data, const Shape& shape, DType dt = DType::F32) {   // creation.rs:25-84
        T t = empty(shape, dt);
        if (!t.size()) return t;
        if (dt == DType::F32) {
            B::h2d(t.buf->ptr, data, t.size() * sizeof(float));
        } else if (dt == DType::BF16) {
            std::vector<uint16_t> v(t.size());
            for (size_t i = 0; i < v.size(); ++i) v[i] = f32_to_bf16(data[i]);
            B::h2d(t.buf->ptr, v.data(), v.size() * 2);
        } else {
            throw Error(ErrKind::UnsupportedDType, "from_host: needs a float dtype");
        }
        return t;
    }
    static T share_buffer(const T& s) {                                             // creation.rs:86-102
        T t;
        t.buf = s.buf;
        t.layout = s.layout;
        t.dtype = s.dtype;
        return t;
    }

    // -- reading back --
    std::vector<float> to_vec() const {                                            // logical order
        T c = contiguous();
        std::vector<float> out(c.size());
        if (!c.size()) return out;
        const size_t esz = dtype_size(c.dtype);
        const char* src = (const char*)c.buf->ptr + c.offset() * esz;
        if (c.dtype == DType::F32) {
            B::d2h(out.data(), src, c.size() * 4);
        } else if (c.dtype == DType::BF16) {
            std::vector<uint16_t> raw(c.size());
            B::d2h(raw.data(), src, c.size() * 2);
            for (size_t i = 0; i < raw.size(); ++i) out[i] = bf16_to_f32(raw[i]);
        } else {
            std::vector<uint8_t> raw(c.size());
            B::d2h(raw.data(), src, c.size());
            for (size_t i = 0; i < raw.size(); ++i) out[i] = raw[i] ? 1.0f : 0.0f;
        }
        return out;
    }
    float item() const {                                                            // buffer/mod.rs:596-614
        if (size() != 1) throw Error(ErrKind::InvalidShape, "item() needs a tensor with one element");
        if (dtype == DType::F32) {
            float v;
            B::d2h(&v, (const char*)buf->ptr + offset() * 4, 4);
            return v;
        }
        if (dtype == DType::BF16) {
            uint16_t v;
            B::d2h(&v, (const char*)buf->ptr + offset() * 2, 2);
            return bf16_to_f32(v);
        }
        throw Error(ErrKind::UnsupportedDType, "item() of a bool tensor");
    }

    // -- grad plumbing (wt.rs:92-104, lib.rs:213-285) --
    void with_grad() {
        if (!is_float(dtype)) throw Error(ErrKind::UnsupportedDType, "with_grad needs a float tensor");
        requires_grad = true;
        if (!grad_cell) {
            grad_cell = std::make_shared<GradCell<B>>();
            grad_cell->shape = shape();
            grad_cell->dtype = dtype;
        }
    }
    bool has_grad() const { return (bool)grad_cell; }
    T grad() const {
        if (!has_grad()) throw Error(ErrKind::InvalidOperation, "tensor has no grad");
        if (!grad_cell->g) grad_cell->g = std::make_shared<T>(zeros(grad_cell->shape, grad_cell->dtype));
        return *grad_cell->g;
    }
    void accumulate_grad(const T& g) const {                                        // lib.rs:221-241
        if (!has_grad()) return;
        // The first gradient of a tensor is added into zeros.  When it is itself a fresh buffer of sums that started
        // from +0 (an identity sum_to_shape in a binary op's backward), `0 + g` would be a copy of it bit for bit: the
        // buffer becomes the gradient as it is.  (Nobody else holds it: the caller's vector of gradients does, and
        // only reads it.)
        if (autograd_shortcuts() && !grad_cell->g && g.sums_from_zero && g.buf.use_count() == 1 && g.dtype == grad_cell->dtype &&
            g.is_contiguous() && g.offset() == 0 && g.shape() == grad_cell->shape) {
            grad_cell->g = std::make_shared<T>(share_buffer(g));
            return;
        }
        // (a view qualifies when every element it addresses lies inside the first size() elements of its buffer: the
        // strided sum_to_shape kernel wraps source indices at num_els, reduction.rs:112-140, and must not get to)
        auto inside = [](const T& v) {
            size_t last = v.offset();
            for (size_t i = 0; i < v.ndim(); ++i) last += (v.shape()[i] ? v.shape()[i] - 1 : 0) * v.strides()[i];
            return last < v.size();
        };
        if (!grad_cell->g && g.dtype == grad_cell->dtype && g.shape() == grad_cell->shape &&
            (g.is_contiguous() || (autograd_shortcuts() && g.size() && inside(g)))) {
            T fresh = empty(grad_cell->shape, g.dtype);
            auto md = meta_to_shape(g, g.shape());
            by_dtype(g.dtype, "accumulate_grad", [&](auto tag) {
                using E = typename decltype(tag)::type;
                K<E>::sum_to_shape(g.size(), g.ndim(), md.data(), g.template p<E>(), fresh.template p<E>());      // fresh = 0 + g
            });
            ++backend_calls();
            B::check();
            grad_cell->g = std::make_shared<T>(fresh);
            return;
        }
        if (!grad_cell->g) grad_cell->g = std::make_shared<T>(zeros(grad_cell->shape, grad_cell->dtype));
        grad_cell->g->add_(g);
    }
    T detach() const {                                                              // f.rs:67-73
        T r = *this;
        r.requires_grad = false;
        r.node.reset();
        return r;
    }
    void zero_grad() const {                                                        // lib.rs:243-285
        std::unordered_set<const void*> visited;
        zero_grad_impl(visited);
    }
    void zero_grad_impl(std::unordered_set<const void*>& visited) const {
        if (!visited.insert(buf.get()).second) return;
        if (has_grad()) grad_cell->g.reset();                       // all zeros again
        if (node)
            for (const T& in : node->inputs)
                if (in.requires_grad) in.zero_grad_impl(visited);
    }
    void backward() const {                                                         // lib.rs:293-301
        if (!requires_grad) return;
        // (a one-element loss whose node takes the seed as a constant: no fill, and nothing for its backward pass to wait for)
        T go;
        if (autograd_shortcuts() && node && node->takes_unit_seed && size() == 1) {
            go.layout = layout;
            go.dtype = dtype;
            go.unit_seed = true;
        } else {
            go = ones_like(*this);
        }
        BackwardScope scope;
        std::unordered_set<const void*> visited;
        backward_tracking(go, visited);
    }
    // The walk keys "visited" on the buffer, so views of one buffer count as one tensor (lib.rs:308-323).
    void backward_tracking(const T& go, std::unordered_set<const void*>& visited) const {
        if (!visited.insert(buf.get()).second) return;
        if (!node || !node->backward) return;
        std::vector<T> grads = node->backward(node->inputs, go);                    // lib.rs:93-111
        for (size_t i = 0; i < node->inputs.size(); ++i) {
            const T& in = node->inputs[i];
            // (a closure that already added its gradient into the input's - a leaf's - hands back a tensor without a buffer)
            if (in.requires_grad && i < grads.size() && grads[i].buf) {
                in.accumulate_grad(grads[i]);
                in.backward_tracking(grads[i], visited);
            }
        }
    }
    void set_node(const char* op, std::vector<T> inputs, BackwardFn fn) {
        node = std::make_shared<Node<B>>();
        node->op = op;
        node->inputs = std::move(inputs);
        node->backward = std::move(fn);
    }

    // -- metadata builders --
    static std::vector<size_t> meta_binary(const T& l, const T& r) {                // ops/binary.rs:754-769
        std::vector<size_t> m(l.shape());
        m.insert(m.end(), l.strides().begin(), l.strides().end());
        m.insert(m.end(), r.strides().begin(), r.strides().end());
        m.push_back(l.offset());
        m.push_back(r.offset());
        return m;
    }
    static std::vector<size_t> meta_unary(const T& t) {                             // ops/unary.rs:1309-1320
        std::vector<size_t> m(t.shape());
        m.insert(m.end(), t.strides().begin(), t.strides().end());
        m.push_back(t.offset());
        return m;
    }
    static std::vector<size_t> meta_reduce(const T& t, size_t dim) {                // ops/reduction.rs:722-732
        std::vector<size_t> m(t.shape());
        m.insert(m.end(), t.strides().begin(), t.strides().end());
        m.push_back(t.shape()[dim]);
        m.push_back(t.strides()[dim]);
        m.push_back(t.offset());
        return m;
    }
    static std::vector<size_t> meta_to_shape(const T& t, const Shape& target) {     // ops/reduction.rs:734-743
        std::vector<size_t> m(t.shape());
        m.insert(m.end(), t.strides().begin(), t.strides().end());
        m.insert(m.end(), target.begin(), target.end());
        m.push_back(t.offset());
        return m;
    }

    void need_f32(const char* what) const {
        if (dtype != DType::F32) throw Error(ErrKind::UnsupportedDType, std::string(what) + ": only f32 tensors are supported");
    }

    // -- binary ops (ops/binary.rs:11-215) --
    static std::pair<T, T> broadcast_tensors(const T& a, const T& b) {              // utils/broadcast.rs:4-31
        size_t an = a.ndim(), bn = b.ndim(), on = std::max(an, bn);
        Shape out(on);
        for (size_t i = 0; i < on; ++i) {
            size_t ad = i < an ? a.shape()[an - 1 - i] : 1, bd = i < bn ? b.shape()[bn - 1 - i] : 1;
            if (ad == 1 || bd == 1 || ad == bd) out[on - 1 - i] = std::max(ad, bd);
            else throw Error(ErrKind::InvalidShape, "Cannot broadcast shapes " + shape_str(a.shape()) + " and " + shape_str(b.shape()));
        }
        // A 0-d operand is materialised by the reference (broadcast_scalar_to: item() and a host fill); the kernels read a
        // view with zero strides just as well, and the result is the same bits.
        auto spread = [&](const T& t) {
            if (!autograd_shortcuts() || !t.shape().empty() || out.empty()) return t.broadcast(out);
            T v = share_buffer(t);
            v.layout = t.layout.broadcast_to(out);
            if (t.requires_grad) v.with_grad();
            return v;
        };
        return {spread(a), spread(b)};
    }
    // promote both sides to the common dtype, broadcast, run the kernel (ops/binary.rs:17-44)
    T binary_forward(const T& rhs_in, BinOp op, T& lhs_b, T& rhs_b) const {
        if (!is_float(dtype) || !is_float(rhs_in.dtype)) throw Error(ErrKind::UnsupportedDType, "binary op: needs float tensors");
        const DType dt = promoted(dtype, rhs_in.dtype);
        auto pr = broadcast_tensors(to_dtype(dt), rhs_in.to_dtype(dt));
        lhs_b = pr.first;
        rhs_b = pr.second;
        T result = empty(lhs_b.shape(), dt);
        auto md = meta_binary(lhs_b, rhs_b);
        by_dtype(dt, "binary op", [&](auto tag) {
            using E = typename decltype(tag)::type;
            K<E>::bin[op](lhs_b.size(), lhs_b.ndim(), md.data(), lhs_b.template p<E>(), rhs_b.template p<E>(), result.template p<E>());
        });
        ++backend_calls();
        B::check();
        return result;
    }
    // backward_tracking only looks at the gradient of an input that requires one
    static bool wanted(const std::vector<T>& inputs, size_t i) { return !autograd_shortcuts() || inputs[i].requires_grad; }
    T add(const T& rhs) const {                                                     // ops/binary.rs:11-60
        T l, r;
        T result = binary_forward(rhs, ADD, l, r);
        if (requires_grad || r.requires_grad) {
            result.with_grad();
            Shape ls = shape(), rs = rhs.shape();
            result.set_node("add", {*this, rhs}, [ls, rs](const std::vector<T>& in, const T& go) {
                return std::vector<T>{wanted(in, 0) ? go.sum_to_shape(ls) : T(), wanted(in, 1) ? go.sum_to_shape(rs) : T()};
            });
        }
        return result;
    }
    T sub(const T& rhs) const {                                                     // ops/binary.rs:62-111
        T l, r;
        T result = binary_forward(rhs, SUB, l, r);
        if (requires_grad || r.requires_grad) {
            result.with_grad();
            Shape ls = shape(), rs = rhs.shape();
            result.set_node("sub", {*this, rhs}, [ls, rs](const std::vector<T>& in, const T& go) {
                return std::vector<T>{wanted(in, 0) ? go.sum_to_shape(ls) : T(), wanted(in, 1) ? go.neg().sum_to_shape(rs) : T()};
            });
        }
        return result;
    }
    T mul(const T& rhs) const {                                                     // ops/binary.rs:113-164
        T l, r;
        T result = binary_forward(rhs, MUL, l, r);
        if (requires_grad || r.requires_grad) {
            result.with_grad();
            Shape ls = shape(), rs = rhs.shape();
            result.set_node("mul", {*this, rhs}, [ls, rs, l, r](const std::vector<T>& in, const T& go) {
                return std::vector<T>{wanted(in, 0) ? go.mul(r).sum_to_shape(ls) : T(), wanted(in, 1) ? go.mul(l).sum_to_shape(rs) : T()};
            });
        }
        return result;
    }
    T div(const T& rhs) const {                                                     // ops/binary.rs:166-222
        T l, r;
        T result = binary_forward(rhs, DIV, l, r);
        if (requires_grad || r.requires_grad) {
            result.with_grad();
            Shape ls = shape(), rs = rhs.shape();
            result.set_node("div", {*this, rhs}, [ls, rs, l, r](const std::vector<T>& in, const T& go) {
                return std::vector<T>{wanted(in, 0) ? go.div(r).sum_to_shape(ls) : T(),
                                      wanted(in, 1) ? go.mul(l).div(r.square()).neg().sum_to_shape(rs) : T()};
            });
        }
        return result;
    }
    void inplace(const T& rhs_in, InplaceOp op) {                                   // ops/binary.rs:653-700
        T rhs = shape() == rhs_in.shape() ? rhs_in : rhs_in.broadcast(shape());
        if (rhs.dtype != dtype) rhs = rhs.to_dtype(dtype);                          // binary.rs:660-662
        auto md = meta_binary(*this, rhs);
        by_dtype(dtype, "in-place op", [&](auto tag) {
            using E = typename decltype(tag)::type;
            K<E>::inplace[op](size(), ndim(), md.data(), this->template p<E>(), rhs.template p<E>());
        });
        ++backend_calls();
        B::check();
    }
    void add_(const T& rhs) { inplace(rhs, ADD_INPLACE); }
    void sub_(const T& rhs) { inplace(rhs, SUB_INPLACE); }

    // -- unary ops (ops/unary.rs) --
    T unary_forward(UnOp op) const {
        T result = empty(shape(), dtype);
        auto md = meta_unary(*this);
        by_dtype(dtype, "unary op", [&](auto tag) {
            using E = typename decltype(tag)::type;
            K<E>::un[op](size(), ndim(), md.data(), this->template p<E>(), result.template p<E>());
        });
        ++backend_calls();
        B::check();
        return result;
    }
    // `target` is the dtype the reference promotes the tensor to before the kernel runs
    T unary_c_forward(UncOp op, float c, DType target) const {
        if (!is_float(dtype)) throw Error(ErrKind::UnsupportedDType, "scalar op: needs a float tensor");
        T input = to_dtype(target);
        T result = empty(shape(), target);
        auto md = meta_unary(input);
        by_dtype(target, "scalar op", [&](auto tag) {
            using E = typename decltype(tag)::type;
            K<E>::unc[op](input.size(), input.ndim(), md.data(), input.template p<E>(), scalar_as<E>(c), result.template p<E>());
        });
        ++backend_calls();
        B::check();
        return result;
    }
    DType scalar_target(float c) const { return integer_valued(c) ? dtype : DType::F32; }
    T neg() const {                                                                 // ops/unary.rs:8-43
        T result = unary_forward(NEG);
        if (requires_grad) {
            result.with_grad();
            result.set_node("neg", {*this}, [](const std::vector<T>&, const T& go) { return std::vector<T>{go.neg()}; });
        }
        return result;
    }
    T square() const {                                                              // ops/unary.rs:112-147
        T result = unary_forward(SQUARE);
        if (requires_grad) {
            result.with_grad();
            T input = *this;
            result.set_node("square", {*this}, [input](const std::vector<T>&, const T& go) {
                return std::vector<T>{go.mul_scalar(2.0f).mul(input)};
            });
        }
        return result;
    }
    T sqrt() const {                                                                // ops/unary.rs:149-184
        if (!is_float(dtype)) throw Error(ErrKind::UnsupportedDType, "sqrt: needs a float tensor");
        T result = unary_forward(SQRT);
        if (requires_grad) {
            result.with_grad();
            T output = result;
            result.set_node("sqrt", {*this}, [output](const std::vector<T>&, const T& go) {
                return std::vector<T>{go.div(output.mul_scalar(2.0f))};
            });
        }
        return result;
    }
    T relu() const {                                                                // ops/unary.rs:186-222
        T result = unary_forward(RELU);
        if (requires_grad) {
            result.with_grad();
            T input = *this;
            result.set_node("relu", {*this}, [input](const std::vector<T>&, const T& go) {
                return std::vector<T>{go.mul(input.gt_scalar(0.0f).to_dtype(input.dtype))};
            });
        }
        return result;
    }
    T tanh() const {                                                                // ops/unary.rs:261-296
        T result = unary_forward(TANH);
        if (requires_grad) {
            result.with_grad();
            T output = result;
            result.set_node("tanh", {*this}, [output](const std::vector<T>&, const T& go) {
                return std::vector<T>{go.mul(output.pow(2.0f).neg().add_scalar(1.0f))};
            });
        }
        return result;
    }
    T gelu() const {                                                                // ops/unary.rs:298-351
        T result = unary_forward(GELU);
        if (requires_grad) {
            result.with_grad();
            T input = *this;
            result.set_node("gelu", {*this}, [input](const std::vector<T>&, const T& go) {
                const float c0 = 0.7978845608028654f, coeff = 0.044715f;
                T x2 = input.mul(input);
                T x3 = x2.mul(input);
                T tanh_arg = input.add(x3.mul_scalar(coeff)).mul_scalar(c0);
                T tanh_val = tanh_arg.tanh();
                T sech2 = tanh_val.mul(tanh_val).mul_scalar(-1.0f).add_scalar(1.0f);
                T inner = x2.mul_scalar(3.0f * coeff).add_scalar(1.0f).mul_scalar(c0);
                T term1 = tanh_val.add_scalar(1.0f).mul_scalar(0.5f);
                T term2 = input.mul(sech2).mul(inner).mul_scalar(0.5f);
                return std::vector<T>{go.mul(term1.add(term2))};
            });
        }
        return result;
    }
    T exp() const {                                                                 // ops/unary.rs:583-618
        T result = unary_forward(EXP);
        if (requires_grad) {
            result.with_grad();
            T output = result;
            result.set_node("exp", {*this}, [output](const std::vector<T>&, const T& go) { return std::vector<T>{go.mul(output)}; });
        }
        return result;
    }
    T add_scalar(float c) const {                                                   // ops/unary.rs:794-830
        T result = unary_c_forward(ADD_SCALAR, c, scalar_target(c));
        if (requires_grad) {
            result.with_grad();
            result.set_node("add_scalar", {*this}, [](const std::vector<T>&, const T& go) { return std::vector<T>{go}; });
        }
        return result;
    }
    T mul_scalar(float c) const {                                                   // ops/unary.rs:870-907
        T result = unary_c_forward(MUL_SCALAR, c, scalar_target(c));
        if (requires_grad) {
            result.with_grad();
            result.set_node("mul_scalar", {*this}, [c](const std::vector<T>&, const T& go) { return std::vector<T>{go.mul_scalar(c)}; });
        }
        return result;
    }
    T div_scalar(float c) const {                                                   // ops/unary.rs:909-946
        T result = unary_c_forward(DIV_SCALAR, c, dtype);
        if (requires_grad) {
            result.with_grad();
            result.set_node("div_scalar", {*this}, [c](const std::vector<T>&, const T& go) { return std::vector<T>{go.div_scalar(c)}; });
        }
        return result;
    }
    T pow(float e) const {                                                          // ops/unary.rs:1042-1082
        T result = unary_c_forward(POW, e, scalar_target(e));
        if (requires_grad) {
            result.with_grad();
            T input = *this;
            result.set_node("pow", {*this}, [input, e](const std::vector<T>&, const T& go) {
                // (powf(x, 1) is x)
                return std::vector<T>{go.mul_scalar(e).mul(autograd_shortcuts() && e - 1.0f == 1.0f ? input : input.pow(e - 1.0f))};
            });
        }
        return result;
    }
    T gt_scalar(float c) const {                                                    // ops/unary.rs:1264-1284 (bool result, no grad)
        T result = empty(shape(), DType::BOOL);
        auto md = meta_unary(*this);
        by_dtype(dtype, "gt_scalar", [&](auto tag) {
            using E = typename decltype(tag)::type;
            K<E>::gt_scalar(size(), ndim(), md.data(), this->template p<E>(), scalar_as<E>(c), (uint8_t*)result.buf->ptr);
        });
        ++backend_calls();
        B::check();
        return result;
    }
    // with_dtype (wt.rs:65-84): the whole buffer is converted, the layout stays; a clone of the tensor otherwise
    // (promote_tensor, utils/promotion.rs:62-73), so requires_grad, the gradient and the node travel with it
    T to_dtype(DType target) const {
        if (dtype == target) return *this;
        T r = *this;
        r.dtype = target;
        r.buf = std::make_shared<Storage<B>>(buf->len, target);
        const size_t n = buf->len;
        if (dtype == DType::BOOL && target == DType::F32) K<float>::cast_from_bool(n, (const uint8_t*)buf->ptr, r.template p<float>());
        else if (dtype == DType::BOOL && target == DType::BF16) K<uint16_t>::cast_from_bool(n, (const uint8_t*)buf->ptr, r.template p<uint16_t>());
        else if (dtype == DType::BF16 && target == DType::F32) B::cast_bf16_f32(n, p<uint16_t>(), r.template p<float>());
        else if (dtype == DType::F32 && target == DType::BF16) B::cast_f32_bf16(n, p<float>(), r.template p<uint16_t>());
        else throw Error(ErrKind::UnsupportedDType, "to_dtype: unsupported conversion");
        ++cast_calls();
        B::check();
        return r;
    }

    // -- reductions (ops/reduction.rs) --
    size_t norm_dim(int dim, size_t nd, bool allow_end = false) const {
        long d = dim < 0 ? (long)nd + dim : dim;
        if (d < 0 || (size_t)d >= nd + (allow_end ? 1 : 0))
            throw Error(ErrKind::DimensionOutOfBounds, "dimension " + std::to_string(dim) + " out of bounds for " + std::to_string(nd) + " dims");
        return (size_t)d;
    }
    T reduce_forward(RedOp op, size_t dim, bool keep_dim) const {
        Shape out = shape();
        out.erase(out.begin() + dim);
        T result = empty(out, dtype);       // the reference zero-fills first (reduction.rs:28); the kernels write every output
        auto md = meta_reduce(*this, dim);
        by_dtype(dtype, "reduction", [&](auto tag) {
            using E = typename decltype(tag)::type;
            K<E>::red[op](size(), ndim(), 1, md.data(), this->template p<E>(), result.template p<E>());
        });
        ++backend_calls();
        B::check();
        result.sums_from_zero = op == SUM;
        if (keep_dim) {
            Shape ks = shape();
            ks[dim] = 1;
            result = result.view(ks);
        }
        return result;
    }
    T sum(int dim_in, bool keep_dim) const {                                        // ops/reduction.rs:9-74
        size_t dim = norm_dim(dim_in, ndim());
        // (inside backward(): the sum over an axis of length 1 is `0 + x`; of sums that started from +0 that is x itself)
        if (autograd_shortcuts() && backward_depth() > 0 && !requires_grad && sums_from_zero && shape()[dim] == 1 && is_contiguous()) {
            Shape ns = shape();
            if (!keep_dim) ns.erase(ns.begin() + dim);
            return view_like("sum", ns);
        }
        T result = reduce_forward(SUM, dim, keep_dim);
        if (requires_grad) {
            result.with_grad();
            Shape in_shape = shape();
            result.set_node("sum", {*this}, [in_shape, dim, keep_dim](const std::vector<T>&, const T& go) {
                if (keep_dim) return std::vector<T>{go.broadcast(in_shape)};
                Shape gs = in_shape;
                gs[dim] = 1;
                return std::vector<T>{go.reshape(gs).broadcast(in_shape)};
            });
        }
        return result;
    }
    T sum_all() const {                                                             // ops/reduction.rs:76-83
        // The reference sums one dim after the other, innermost first: n kernels forward and n small broadcasts and
        // accumulations backward.  A contiguous f32 tensor is summed in one sum_to_shape call to [1, .., 1] instead (the
        // MLP's own `[10000,1] -> []` is such a call); every gradient is the same bytes, the sum itself is added up in
        // another order (within the f32 tolerance of a reduction either way).
        if (sum_all_in_one_pass() && dtype == DType::F32 && ndim() >= 2 && size() > 0 && is_contiguous() && offset() == 0) {
            // (a node of its own: a view of a [1, .., 1] result would share that result's buffer, and backward() takes
            // tensors that share a buffer for one tensor, lib.rs:308-323)
            const Shape ones(ndim(), 1);
            T result = empty(Shape{}, dtype);
            auto md = meta_to_shape(*this, ones);
            K<float>::sum_to_shape(size(), ndim(), md.data(), this->template p<float>(), result.template p<float>());
            ++backend_calls();
            B::check();
            if (requires_grad) {
                result.with_grad();
                Shape in_shape = shape();
                result.set_node("sum_all", {*this}, [in_shape, ones](const std::vector<T>&, const T& go) {
                    return std::vector<T>{go.reshape(ones).broadcast(in_shape)};
                });
            }
            return result;
        }
        T result = *this;
        for (size_t d = ndim(); d-- > 0;) result = result.sum((int)d, false);
        return result;
    }
    T sum_to_shape(const Shape& target) const {                                     // ops/reduction.rs:85-143
        if (target.size() != ndim()) {
            if (ndim() > target.size()) {
                T result = *this;
                while (result.ndim() > target.size()) result = result.sum(0, false);
                return result.sum_to_shape(target);
            }
            throw Error(ErrKind::ShapeMismatch, "Target shape has more dimensions than input");
        }
        for (size_t i = 0; i < target.size(); ++i)
            if (target[i] == 0 || shape()[i] % target[i] != 0)
                throw Error(ErrKind::ShapeMismatch, "Dimension " + std::to_string(i) + " is not divisible: " + std::to_string(shape()[i]) +
                                                        " -> " + std::to_string(target[i]));
        // (inside backward(): `0 + x` of sums that started from +0 is x)
        if (autograd_shortcuts() && backward_depth() > 0 && !requires_grad && sums_from_zero && shape() == target) return *this;
        T result = empty(target, dtype);    // zero-filled in the reference (reduction.rs:112); fully written by the kernel
        auto md = meta_to_shape(*this, target);
        by_dtype(dtype, "sum_to_shape", [&](auto tag) {
            using E = typename decltype(tag)::type;
            K<E>::sum_to_shape(size(), ndim(), md.data(), this->template p<E>(), result.template p<E>());
        });
        ++backend_calls();
        B::check();
        result.sums_from_zero = true;
        if (requires_grad) {
            result.with_grad();
            Shape in_shape = shape();
            result.set_node("sum_to_shape", {*this}, [in_shape](const std::vector<T>&, const T& go) { return std::vector<T>{go.broadcast(in_shape)}; });
        }
        return result;
    }
    T mean(int dim_in, bool keep_dim) const {                                       // ops/reduction.rs:145-216
        size_t dim = norm_dim(dim_in, ndim());
        T result = reduce_forward(MEAN, dim, keep_dim);
        if (requires_grad) {
            result.with_grad();
            Shape in_shape = shape();
            size_t dim_size = shape()[dim];
            result.set_node("sum", {*this}, [in_shape, dim, keep_dim, dim_size](const std::vector<T>&, const T& go_in) {
                T go = go_in;
                if (!keep_dim) {
                    Shape gs = in_shape;
                    gs[dim] = 1;
                    go = go.view(gs);
                }
                return std::vector<T>{go.broadcast(in_shape).div_scalar((float)dim_size)};
            });
        }
        return result;
    }
    T mean_all() const {                                                            // ops/reduction.rs:218-225
        T result = *this;
        for (size_t d = ndim(); d-- > 0;) result = result.mean((int)d, false);
        return result;
    }

    // -- views and layout ops (ops/transform.rs) --
    T view_like(const char* op, const Shape& ns) const {
        T result = share_buffer(*this);
        result.layout.view(ns);
        result.sums_from_zero = sums_from_zero && !requires_grad;
        if (requires_grad) {
            result.with_grad();
            Shape orig = shape();
            result.set_node(op, {*this}, [orig](const std::vector<T>&, const T& go) { return std::vector<T>{go.reshape(orig)}; });
        }
        return result;
    }
    Shape shape_with_auto(const std::vector<long>& req) const {                     // ops/transform.rs:381-440
        long product = 1;
        int auto_idx = -1;
        for (size_t i = 0; i < req.size(); ++i) {
            if (req[i] == -1) {
                if (auto_idx >= 0) throw Error(ErrKind::InvalidShape, "Only one dimension can be -1");
                auto_idx = (int)i;
            } else if (req[i] <= 0) {
                throw Error(ErrKind::InvalidShape, "Invalid dimension size: " + std::to_string(req[i]));
            } else {
                product *= req[i];
            }
        }
        Shape out(req.size());
        long total = (long)size();
        if (auto_idx >= 0) {
            if (product == 0) throw Error(ErrKind::InvalidShape, "Cannot infer size for dimension -1");
            long a = total / product;
            if (a * product != total) throw Error(ErrKind::InvalidShape, "Cannot reshape tensor: incompatible dimensions");
            for (size_t i = 0; i < req.size(); ++i) out[i] = (size_t)((int)i == auto_idx ? a : req[i]);
        } else {
            if (product != total) throw Error(ErrKind::InvalidShape, "Total size of new shape must be equal to old size");
            for (size_t i = 0; i < req.size(); ++i) out[i] = (size_t)req[i];
        }
        return out;
    }
    static std::vector<long> as_long(const Shape& s) { return std::vector<long>(s.begin(), s.end()); }
    T view(const Shape& ns) const { return view_like("view", shape_with_auto(as_long(ns))); }   // ops/transform.rs:10-28
    T view(const std::vector<long>& ns) const { return view_like("view", shape_with_auto(ns)); }
    T squeeze(int dim_in) const {                                                   // ops/transform.rs:30-71
        size_t dim = norm_dim(dim_in, ndim());
        if (shape()[dim] != 1) return *this;
        Shape ns = shape();
        ns.erase(ns.begin() + dim);
        if (ns.empty()) ns.push_back(1);          // a squeezed [1] stays [1] (transform.rs:50-52)
        return view_like("squeeze", ns);
    }
    T squeeze_all() const {                                                         // ops/transform.rs:73-92
        Shape ns;
        for (size_t d : shape())
            if (d != 1) ns.push_back(d);
        return view_like("squeeze_all", ns);
    }
    T unsqueeze(int dim_in) const {                                                 // ops/transform.rs:94-128
        size_t dim = norm_dim(dim_in, ndim(), true);
        Shape ns = shape();
        ns.insert(ns.begin() + dim, 1);
        return view_like("unsqueeze", ns);
    }
    T transpose(int d0_in, int d1_in) const {                                       // ops/transform.rs:132-162
        long d0 = d0_in < 0 ? (long)ndim() + d0_in : d0_in, d1 = d1_in < 0 ? (long)ndim() + d1_in : d1_in;
        if (d0 < 0 || d1 < 0) throw Error(ErrKind::DimensionOutOfBounds, "transpose: dimension out of bounds");
        T result = share_buffer(*this);
        result.layout.transpose((size_t)d0, (size_t)d1);
        if (requires_grad) {
            result.with_grad();
            result.set_node("transpose", {*this}, [d0, d1](const std::vector<T>&, const T& go) {
                return std::vector<T>{go.transpose((int)d0, (int)d1)};
            });
        }
        return result;
    }
    T broadcast(const Shape& target) const {                                        // ops/transform.rs:278-316
        if (shape() == target) return *this;
        if (shape().empty()) return broadcast_scalar_to(target);
        if (target.empty()) throw Error(ErrKind::InvalidShape, "Cannot broadcast non-scalar shape " + shape_str(shape()) + " to scalar ()");
        T result = share_buffer(*this);
        result.layout = layout.broadcast_to(target);
        if (requires_grad) {
            result.with_grad();
            Shape orig = shape();
            result.set_node("broadcast", {*this}, [orig](const std::vector<T>&, const T& go) { return std::vector<T>{go.sum_to_shape(orig)}; });
        }
        return result;
    }
    T broadcast_left(const Shape& batch) const {                                    // ops/transform.rs:322-326
        Shape ns = batch;
        ns.insert(ns.end(), shape().begin(), shape().end());
        return broadcast(ns);
    }
    T broadcast_scalar_to(const Shape& target) const {                              // ops/transform.rs:328-349
        T result = empty(target, dtype);
        by_dtype(dtype, "broadcast", [&](auto tag) {                                // the reference: item() + host fill
            using E = typename decltype(tag)::type;
            K<E>::broadcast_scalar(result.size(), this->template p<E>() + offset(), result.template p<E>());
        });
        if (requires_grad) {
            result.with_grad();
            result.set_node("broadcast_scalar", {*this}, [](const std::vector<T>&, const T& go) { return std::vector<T>{go.sum_all()}; });
        }
        return result;
    }
    T contiguous() const {                                                          // f.rs:11-41
        if (is_contiguous()) return *this;
        T result = empty(shape(), dtype);
        auto md = meta_unary(*this);
        // bool tensors only come out of comparisons and are contiguous there
        by_dtype(dtype, "contiguous", [&](auto tag) {
            using E = typename decltype(tag)::type;
            K<E>::copy_strided(size(), ndim(), md.data(), this->template p<E>(), result.template p<E>());
        });
        return result;
    }
    T reshape(const std::vector<long>& req) const {                                 // ops/transform.rs:353-388
        Shape ns = shape_with_auto(req);
        if (is_contiguous()) return view_like("reshape", ns);
        T result = contiguous();
        result.layout.view(ns);
        if (requires_grad) {           // node without with_grad, as the reference has it: gradients stop here
            Shape orig = shape();
            result.set_node("reshape", {*this}, [orig](const std::vector<T>&, const T& go) { return std::vector<T>{go.reshape(orig)}; });
        }
        return result;
    }
    T reshape(const Shape& ns) const { return reshape(as_long(ns)); }

    // -- matmul (ops/matmul.rs:11-157) --
    static std::pair<std::vector<size_t>, Shape> meta_matmul(const T& a, const T& b) {   // ops/matmul.rs:227-264
        Shape as = a.shape(), bs = b.shape(), ast = a.strides(), bst = b.strides();
        if (as.size() == 1) {
            as.insert(as.begin(), 1);
            ast.insert(ast.begin(), ast[0] * as[1]);
        }
        if (bs.size() == 1) {
            bs.push_back(1);
            bst.push_back(1);
        }
        size_t on = as.size();
        Shape out(as.begin(), as.end() - 2);
        out.push_back(as[on - 2]);
        out.push_back(bs[on - 1]);
        std::vector<size_t> m{on, as.size(), bs.size()};
        m.insert(m.end(), out.begin(), out.end());
        m.insert(m.end(), as.begin(), as.end());
        m.insert(m.end(), bs.begin(), bs.end());
        m.insert(m.end(), ast.begin(), ast.end());
        m.insert(m.end(), bst.begin(), bst.end());
        m.push_back(a.offset());
        m.push_back(b.offset());
        return {m, out};
    }
    static std::pair<T, T> unify_matmul_shapes(const T& a, const T& b) {            // ops/matmul.rs:161-194
        T ae = a.ndim() == 1 ? a.unsqueeze(0) : a;
        T be = b.ndim() == 1 ? b.unsqueeze((int)b.ndim()) : b;
        size_t an = ae.ndim(), bn = be.ndim();
        if (an < 2 || bn < 2) throw Error(ErrKind::InvalidShape, "matmul: both inputs must have at least 2D after expand");
        size_t M = ae.shape()[an - 2], Ka = ae.shape()[an - 1], Kb = be.shape()[bn - 2], N = be.shape()[bn - 1];
        if (Ka != Kb) throw Error(ErrKind::InvalidShape, "Incompatible shapes for matmul (K mismatch): " + std::to_string(Ka) + " vs " + std::to_string(Kb));
        size_t al = an - 2, bl = bn - 2, ml = std::max(al, bl);
        Shape lead(ml);
        for (size_t i = 0; i < ml; ++i) {                                            // ops/matmul.rs:196-218
            size_t ad = i < al ? ae.shape()[al - 1 - i] : 1, bd = i < bl ? be.shape()[bl - 1 - i] : 1;
            if (ad != bd && ad != 1 && bd != 1)
                throw Error(ErrKind::InvalidShape, "Cannot broadcast leading dims: mismatch " + std::to_string(ad) + " vs " + std::to_string(bd));
            lead[ml - 1 - i] = std::max(ad, bd);
        }
        Shape as = lead, bs = lead;
        as.push_back(M); as.push_back(Ka);
        bs.push_back(Kb); bs.push_back(N);
        return {ae.broadcast(as), be.broadcast(bs)};
    }
    T matmul(const T& rhs_in) const {
        if (!is_float(dtype) || !is_float(rhs_in.dtype)) throw Error(ErrKind::UnsupportedDType, "matmul: needs float tensors");
        const DType dt = promoted(dtype, rhs_in.dtype);                              // ops/matmul.rs:18-30
        size_t ln = ndim(), rn = rhs_in.ndim();
        auto pr = unify_matmul_shapes(to_dtype(dt), rhs_in.to_dtype(dt));
        const T &lhs = pr.first, &rhs = pr.second;
        auto mm = meta_matmul(lhs, rhs);
        T result = empty(mm.second, dt);
        by_dtype(dt, "matmul", [&](auto tag) {
            using E = typename decltype(tag)::type;
            K<E>::matmul(result.size(), mm.first.data(), lhs.template p<E>(), rhs.template p<E>(), result.template p<E>());
        });
        ++backend_calls();
        B::check();
        result.sums_from_zero = true;       // every output is +0 plus its products
        if (ln == 1 && rn == 1) result = result.squeeze_all();
        else if (ln == 1 && rn >= 2) { int d = (int)result.ndim() - 2; if (result.shape()[d] == 1) result = result.squeeze(d); }
        else if (ln >= 2 && rn == 1) { int d = (int)result.ndim() - 1; if (result.shape()[d] == 1) result = result.squeeze(d); }
        if (requires_grad || rhs.requires_grad) {
            result.with_grad();
            result.set_node("matmul", {*this, rhs_in}, [](const std::vector<T>& in, const T& go_in) {     // ops/matmul.rs:63-146
                const DType dt = promoted(promoted(in[0].dtype, in[1].dtype), go_in.dtype);
                const T l = in[0].to_dtype(dt), r = in[1].to_dtype(dt), go = go_in.to_dtype(dt);
                auto mm = meta_matmul(l, r);
                // (zeros_like in the reference; both are fully written.  The backend leaves out a gradient whose buffer is
                // null: the one of an input that requires none - the data a first layer multiplies - is not made)
                const bool want_l = wanted(in, 0), want_r = wanted(in, 1);
                T gl = want_l ? empty(l.shape(), dt) : T(), gr = want_r ? empty(r.shape(), dt) : T();
                by_dtype(dt, "matmul backward", [&](auto tag) {
                    using E = typename decltype(tag)::type;
                    K<E>::matmul_backward(l.size(), r.size(), mm.first.data(), go.template p<E>(), l.template p<E>(), r.template p<E>(),
                                          want_l ? gl.template p<E>() : nullptr, want_r ? gr.template p<E>() : nullptr);
                });
                ++backend_calls();
                B::check();
                gl.sums_from_zero = want_l;
                gr.sums_from_zero = want_r;
                // the gradients go back in the inputs' own dtypes (matmul.rs:137-143)
                return std::vector<T>{want_l ? gl.to_dtype(in[0].dtype) : T(), want_r ? gr.to_dtype(in[1].dtype) : T()};
            });
        }
        return result;
    }
};

template <class B>
struct Node {
    std::string op;
    std::vector<Tensor<B>> inputs;
    typename Tensor<B>::BackwardFn backward;
    bool takes_unit_seed = false;      // the closure handles a Tensor::unit_seed gradient (all ones, no buffer)
};

// ---- seeded normal values (the reference's randn draws from an unseeded thread_rng, creation.rs:318-331) ----
struct SplitMix64 {
    uint64_t s;
    explicit SplitMix64(uint64_t seed) : s(seed) {}
    uint64_t next() {
        uint64_t z = (s += 0x9E3779B97F4A7C15ull);
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        return z ^ (z >> 31);
    }
    double uniform() { return ((next() >> 11) + 0.5) * (1.0 / 9007199254740992.0); }   // (0, 1)
    float normal() {                                                                    // Box-Muller, one value per pair
        double u1 = uniform(), u2 = uniform();
        return (float)(std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586 * u2));
    }
};
template <class B>
Tensor<B> randn(const Shape& shape, uint64_t seed) {
    SplitMix64 g(seed);
    std::vector<float> v(shape_size(shape));
    for (float& x : v) x = g.normal();
    return Tensor<B>::from_host(v.data(), shape);
}

// ---- nn ---------------------------------------------------------------------------------------------
template <class B>
struct Linear {                                                                     // nn/layers/linear.rs:11-98
    using T = Tensor<B>;
    T weight;                 // [out_features, in_features]
    bool has_bias = false;
    T bias;                   // 0-d tensor, as the reference creates it (linear.rs:44)
    // The reference scales neither tensor: the result of mul_scalar(k) is dropped (linear.rs:40,46).
    Linear(size_t in_f, size_t out_f, bool with_bias, uint64_t seed) {
        weight = randn<B>({out_f, in_f}, seed);
        weight.with_grad();
        if (with_bias) {
            bias = randn<B>({}, seed + 1);
            bias.with_grad();
            has_bias = true;
        }
    }
    Linear(const T& w, const T* b) : weight(w) {
        weight.with_grad();
        if (b) { bias = *b; bias.with_grad(); has_bias = true; }
    }
    T forward(const T& input) const {                                               // linear.rs:60-81
        Shape batch;
        if (input.ndim() >= 2) batch.assign(input.shape().begin(), input.shape().end() - 2);
        T w = batch.empty() ? weight : weight.broadcast_left(batch);
        T out = input.matmul(w.transpose(-1, -2));
        return has_bias ? out.add(bias) : out;
    }
    std::vector<T*> parameters() {
        std::vector<T*> p{&weight};
        if (has_bias) p.push_back(&bias);
        return p;
    }
};

template <class B>
struct Conv2d {                                                                     // nn/layers/conv.rs:100-322
    using T = Tensor<B>;
    T weight;                 // [Cout, Cin, kh, kw]
    bool has_bias = false;
    T bias;                   // [Cout]
    size_t kh, kw, sh, sw, ph, pw;
    Conv2d(const T& w, const T* b, size_t kh_, size_t kw_, size_t sh_, size_t sw_, size_t ph_, size_t pw_)
        : weight(w), kh(kh_), kw(kw_), sh(sh_), sw(sw_), ph(ph_), pw(pw_) {
        weight.with_grad();
        if (b) { bias = *b; bias.with_grad(); has_bias = true; }
    }
    // The caller writes stride then padding into slots 8..11 (conv.rs:352-365); the kernel reads them as
    // padding then stride (crates/maidenx_cpu/src/nn/conv.rs:31-34).  Kept as is.
    static std::vector<size_t> conv_meta(size_t Bn, size_t C, size_t H, size_t W, size_t kh, size_t kw, size_t oh, size_t ow,
                                         size_t sh, size_t sw, size_t ph, size_t pw) {
        return {Bn, C, H, W, kh, kw, oh, ow, sh, sw, ph, pw};
    }
    T forward(const T& input) const {                                               // conv.rs:185-310
        if (input.ndim() != 4) throw Error(ErrKind::InvalidShape, "Expected 4D input (batch_size, channels, height, width)");
        input.need_f32("conv2d");
        const size_t Bn = input.shape()[0], C = input.shape()[1], H = input.shape()[2], W = input.shape()[3];
        const size_t oh = (H + 2 * ph - kh) / sh + 1, ow = (W + 2 * pw - kw) / sw + 1;
        const size_t kh_ = kh, kw_ = kw, sh_ = sh, sw_ = sw, ph_ = ph, pw_ = pw;
        const Shape& ws = weight.shape();
        T wm = weight.reshape(Shape{ws[0], ws[1] * ws[2] * ws[3]});
        const auto md = conv_meta(Bn, C, H, W, kh, kw, oh, ow, sh, sw, ph, pw);
        const size_t M = Bn * oh * ow, K = C * kh * kw;
        // Whether the two products with the column matrix gather its entries from the input instead of reading a stored
        // copy (the same tiles and the same order of additions): the backend has the call, the index space fits it, and
        // the weight matrix is the [Cout, K] it is multiplied with.
        bool gathered = false;
        if constexpr (B::has_cols_matmul)
            gathered = (conv_gathered_products() == 2 || (conv_gathered_products() == 1 && !input.requires_grad)) && M && K && ws[0] && M * K < ((size_t)1 << 31) && input.size() < ((size_t)1 << 31) &&
                       ws[1] == C && ws[2] == kh && ws[3] == kw && (wm.strides()[0] == 1 || wm.strides()[1] == 1);
        T cols, out;
        bool in_store = false;       // the product's store already made the layout change and the bias add
        if (gathered) {
            if constexpr (B::has_cols_matmul) {
                out = T::empty({M, ws[0]});
                const size_t rs[2] = {wm.strides()[1], wm.strides()[0]};                  // of wm^T: [K, Cout]
                B::cols_matmul(md.data(), 0, input.f32(), wm.f32() + wm.offset(), ws[0], rs, out.f32());
                ++backend_calls();
                B::check();
            }
        } else {
            // im2col (conv.rs:333-376); the input buffer is passed from its start, as the reference passes it
            cols = T::empty({M, K});
            B::im2col(cols.size(), md.data(), input.f32(), cols.f32());
            ++backend_calls();
            B::check();
            // The product, the [B, oh, ow, Cout] -> [B, Cout, oh, ow] change of layout and the bias add as one call where the
            // backend has it and takes the shapes (the same bits: the product's tiles, then the elementwise add).  Only when
            // the layer's own node records the backward (or nothing does): the ops' nodes are not made this way.
            if constexpr (B::has_conv_forward_product) {
                const bool own_node = input.requires_grad || !(weight.requires_grad || (has_bias && bias.requires_grad));
                if (fused_nn_kernels() && has_bias && own_node && wm.is_contiguous() && bias.is_contiguous() && bias.dtype == DType::F32 &&
                    weight.dtype == DType::F32) {
                    T planes = T::empty({Bn, ws[0], oh, ow});
                    if (B::conv_forward_product(M, K, ws[0], oh * ow, cols.f32(), wm.f32() + wm.offset(), bias.f32() + bias.offset(), planes.f32())) {
                        ++backend_calls();
                        B::check();
                        out = planes;
                        // (what matmul and add would have left on the result)
                        if (weight.requires_grad || bias.requires_grad) out.with_grad();
                        in_store = true;
                    }
                }
            }
            if (!in_store) out = cols.matmul(wm.transpose(-1, -2));
        }
        if (!in_store) {
            out = out.reshape(std::vector<long>{(long)Bn, (long)oh, (long)ow, -1});
            out = out.transpose(1, 3).transpose(2, 3);
            if (has_bias) out = out.add(bias.reshape(Shape{1, bias.shape()[0], 1, 1}));
        }
        if (input.requires_grad) {
            std::vector<T> inputs{input, weight};
            if (has_bias) inputs.push_back(bias);
            out.set_node("conv2d", inputs, [=](const std::vector<T>& in, const T& go) {              // conv.rs:236-306
                const T &x = in[0], &w = in[1];
                std::vector<T> grads;
                // conv.rs:249-251 and :276-278 build the same [B*oh*ow, Cout] copy of the gradient twice; it is made once
                T grad_flat;
                if (x.requires_grad || w.requires_grad) {
                    T gr = go.transpose(2, 3).transpose(1, 3);
                    grad_flat = gr.reshape(Shape{go.shape()[0] * oh * ow, go.shape()[1]});
                }
                if (x.requires_grad) {
                    const Shape& ws = w.shape();
                    T wm = w.reshape(Shape{ws[0], ws[1] * ws[2] * ws[3]});
                    // col2im divides by what it reads as the stride, i.e. by the padding the caller stored in
                    // slots 10, 11: with padding 0 the reference panics (division by zero)
                    if (ph_ == 0 || pw_ == 0)
                        throw Error(ErrKind::InvalidOperation, "col2im: division by zero (padding 0 is read as stride 0)");
                    // When x is a leaf whose gradient already exists, backward() would only add the col2im result to it
                    // (lib.rs:221-241): the backend's accumulating form writes grad + (that result) in one pass - the same
                    // sum, then the same add - and nothing is handed back.
                    T* into = nullptr;
                    if constexpr (B::has_col2im_add) {
                        if (fused_nn_kernels() && autograd_shortcuts() && !x.node && x.grad_cell && x.grad_cell->g) {
                            T& g = *x.grad_cell->g;
                            if (g.dtype == DType::F32 && g.is_contiguous() && g.offset() == 0 && g.shape() == x.shape() && ((uintptr_t)g.f32() % 16) == 0)
                                into = &g;
                        }
                    }
                    T gi = into ? T() : T::empty({Bn, C, H, W});                                     // col2im, conv.rs:378-418
                    // col2im is handed num_els = B*C*H*W (conv.rs:391) and reads no column entry at or beyond that flat
                    // index (crates/maidenx_cpu/src/nn/conv.rs:135), i.e. only the first ceil(B*C*H*W / (C*kh*kw)) rows of
                    // grad_cols; the rows below are never read, so the product is made for those leading rows only (each of
                    // them the same arithmetic as in the whole product).
                    T lead = grad_flat;
                    const size_t row_len = ws[1] * ws[2] * ws[3];
                    const size_t n_in = Bn * C * H * W;
                    const size_t used = row_len ? (n_in + row_len - 1) / row_len : 0;
                    if (conv_skip_unread_grad_cols() && grad_flat.is_contiguous() && used < grad_flat.shape()[0]) {
                        lead = T::share_buffer(grad_flat);
                        lead.layout.shape[0] = used;
                    }
                    T grad_cols = lead.matmul(wm);
                    auto md = conv_meta(Bn, C, H, W, kh_, kw_, oh, ow, sh_, sw_, ph_, pw_);
                    if constexpr (B::has_col2im_add) {
                        if (into) B::col2im_add(into->size(), md.data(), grad_cols.f32(), into->f32());
                    }
                    if (!into) B::col2im(n_in, md.data(), grad_cols.f32(), gi.f32());
                    ++backend_calls();
                    B::check();
                    grads.push_back(gi);
                } else {
                    grads.push_back(T::zeros_like(x));
                }
                if (w.requires_grad) {
                    T gw;
                    if (gathered && (grad_flat.strides()[0] == 1 || grad_flat.strides()[1] == 1)) {
                        if constexpr (B::has_cols_matmul) {
                            gw = T::empty({K, grad_flat.shape()[1]});
                            const size_t rs[2] = {grad_flat.strides()[0], grad_flat.strides()[1]};
                            B::cols_matmul(md.data(), 1, x.f32(), grad_flat.f32() + grad_flat.offset(), grad_flat.shape()[1], rs, gw.f32());
                            ++backend_calls();
                            B::check();
                            gw.sums_from_zero = true;       // a matmul's outputs, like the stored way's
                        }
                    } else {
                        T stored = cols;
                        if (gathered) {                      // (a gradient the call cannot take: store the matrix after all)
                            stored = T::empty({M, K});
                            B::im2col(stored.size(), md.data(), x.f32(), stored.f32());
                            ++backend_calls();
                            B::check();
                        }
                        gw = stored.transpose(-1, -2).matmul(grad_flat);
                    }
                    grads.push_back(gw.reshape(Shape{w.shape()[0], w.shape()[1], kh_, kw_}));
                } else {
                    grads.push_back(T::zeros_like(w));
                }
                if (in.size() > 2) {
                    const T& b = in[2];
                    // conv.rs:287-291 sums the gradient over W, H and the batch, one launch and one intermediate each; a
                    // contiguous f32 gradient is summed to [1, Cout, 1, 1] in one sum_to_shape call instead (the sums are
                    // added up in another order, within the f32 tolerance of a reduction either way)
                    if (!b.requires_grad) grads.push_back(T::zeros_like(b));
                    else if (sum_all_in_one_pass() && go.dtype == DType::F32 && go.is_contiguous() && go.offset() == 0 && go.size() > 0)
                        grads.push_back(go.sum_to_shape(Shape{1, go.shape()[1], 1, 1}).reshape(Shape{go.shape()[1]}));
                    else grads.push_back(go.sum(3, false).sum(2, false).sum(0, false));
                }
                return grads;
            });
        }
        return out;
    }
    std::vector<T*> parameters() {
        std::vector<T*> p{&weight};
        if (has_bias) p.push_back(&bias);
        return p;
    }
};

// whether a tensor is a plain f32 block a fused kernel can take: contiguous from the start of a 16-byte aligned buffer
template <class B>
inline bool plain_f32(const Tensor<B>& t) {
    return t.dtype == DType::F32 && t.size() > 0 && t.is_contiguous() && t.offset() == 0 && ((uintptr_t)t.template p<float>() % 16) == 0;
}

template <class B>
Tensor<B> mse_loss(const Tensor<B>& pred, const Tensor<B>& target) {                // nn/losses/mse.rs:21-29
    using T = Tensor<B>;
    if constexpr (B::has_fused_nn) {
        // sub, pow(2), sum_all and div_scalar as one kernel, and their six backward ops as another: the difference is
        // recomputed there instead of stored, every gradient is what the op sequence gives bit for bit
        if (fused_nn_kernels() && plain_f32(pred) && plain_f32(target) && pred.shape() == target.shape()) {
            T loss = T::empty(Shape{}, DType::F32);
            B::mse_loss(pred.size(), pred.template p<float>(), target.template p<float>(), loss.template p<float>());
            ++backend_calls();
            B::check();
            if (pred.requires_grad || target.requires_grad) {
                loss.with_grad();
                loss.set_node("mse_loss", {pred, target}, [](const std::vector<T>& in, const T& go_in) {
                    // (the seed of backward() arrives without a buffer: the kernel then takes the gradient of the loss as 1)
                    const T go = go_in.unit_seed ? go_in : go_in.to_dtype(DType::F32).contiguous();
                    const float* seed = go_in.unit_seed ? nullptr : go.template p<float>() + go.offset();
                    const bool want_p = T::wanted(in, 0), want_t = T::wanted(in, 1);
                    T gp = want_p ? T::empty(in[0].shape(), DType::F32) : T(), gt = want_t ? T::empty(in[1].shape(), DType::F32) : T();
                    if (want_p || want_t) {
                        B::mse_loss_backward(in[0].size(), in[0].template p<float>(), in[1].template p<float>(),
                                             seed, want_p ? gp.template p<float>() : nullptr,
                                             want_t ? gt.template p<float>() : nullptr);
                        ++backend_calls();
                        B::check();
                    }
                    gp.sums_from_zero = want_p;      // `0 + g`, as sub's sum_to_shape leaves it
                    gt.sums_from_zero = want_t;
                    return std::vector<T>{gp, gt};
                });
                loss.node->takes_unit_seed = true;
            }
            return loss;
        }
    }
    Tensor<B> squared = pred.sub(target).pow(2.0f);
    return squared.sum_all().div_scalar((float)squared.size());
}

template <class B>
struct SGD {                                                                        // nn/optimizers/sgd.rs:6-37
    float lr;
    explicit SGD(float lr_) : lr(lr_) {}
    void step(const std::vector<Tensor<B>*>& params) const {
        for (Tensor<B>* p : params) {
            if (!p->has_grad()) continue;
            if constexpr (B::has_fused_nn) {
                // mul_scalar and the in-place sub as one pass: the same two roundings per element
                const Tensor<B> g = p->grad();
                if (fused_nn_kernels() && plain_f32(*p) && plain_f32(g) && g.shape() == p->shape()) {
                    B::sgd_step(p->size(), p->template p<float>(), g.template p<float>(), lr);
                    ++backend_calls();
                    B::check();
                    continue;
                }
            }
            p->sub_(p->grad().mul_scalar(lr));
        }
    }
    void zero_grad(const std::vector<Tensor<B>*>& params) const {
        for (Tensor<B>* p : params) p->zero_grad();
    }
};

// nn/optimizers/adam.rs:6-99.  The hyper-parameters are f64 scalars (what the reference's `Adam::new(0.001, 0.9,
// 0.999, 1e-8)` builds from literals), so the step's scalar arithmetic is f64 and every tensor op receives the
// value rounded to the tensor's dtype.  The bias terms use beta^(t+1): the reference's loop multiplies t times
// starting from beta (:56-61).  With a backend that has the fused kernel, a contiguous f32 parameter takes one
// call instead of the fourteen ops; the results are the same bits (the moments are then updated in place).
template <class B>
struct Adam {
    double lr, beta1, beta2, eps;
    size_t t = 0;
    bool fused = true;
    std::vector<Tensor<B>> m, v;
    Adam(double lr_, double b1, double b2, double eps_) : lr(lr_), beta1(b1), beta2(b2), eps(eps_) {}
    void step(const std::vector<Tensor<B>*>& params) {
        using T = Tensor<B>;
        if (m.empty() || v.empty()) {
            m.clear();
            v.clear();
            for (T* p : params) { m.push_back(T::zeros_like(*p)); v.push_back(T::zeros_like(*p)); }
        }
        if (m.size() != params.size()) throw Error(ErrKind::InvalidArgument, "Adam: the parameter list changed");
        ++t;
        for (size_t i = 0; i < params.size(); ++i) {
            T* p = params[i];
            if (!p->has_grad()) continue;
            T grad = p->grad();
            double b1t = beta1, b2t = beta2;
            for (size_t k = 0; k < t; ++k) { b1t = b1t * beta1; b2t = b2t * beta2; }
            const double c1 = 1.0 - b1t, c2 = 1.0 - b2t, lr_t = lr * std::sqrt(c2) / c1;
            const double omb1 = 1.0 - beta1, omb2 = 1.0 - beta2;
            if constexpr (B::has_fused_adam) {
                auto plain = [](const T& x) { return x.dtype == DType::F32 && x.is_contiguous(); };
                if (fused && plain(*p) && plain(grad) && plain(m[i]) && plain(v[i]) && grad.size() == p->size()) {
                    B::template K<float>::adam_step(p->size(), p->template p<float>(), grad.template p<float>(), m[i].template p<float>(),
                                                    v[i].template p<float>(), (float)beta1, (float)omb1, (float)beta2, (float)omb2, (float)c1,
                                                    (float)c2, (float)eps, (float)lr_t);
                    ++backend_calls();
                    B::check();
                    continue;
                }
            }
            m[i] = m[i].mul_scalar((float)beta1).add(grad.mul_scalar((float)omb1));
            v[i] = v[i].mul_scalar((float)beta2).add(grad.square().mul_scalar((float)omb2));
            T m_hat = m[i].div_scalar((float)c1), v_hat = v[i].div_scalar((float)c2);
            T step = m_hat.div(v_hat.sqrt().add_scalar((float)eps));
            p->sub_(step.mul_scalar((float)lr_t));
        }
    }
    void zero_grad(const std::vector<Tensor<B>*>& params) const {
        for (Tensor<B>* p : params) p->zero_grad();
    }
};

// ---- a step, many times -------------------------------------------------------------------------------
// Calls step(e) for e = 0 .. epochs-1, or does the same work by replaying a recording of it.
//
// A step on small tensors is launch-bound (tens of small kernels), so when the backend can record graphs it is recorded
// once and replayed: the pool hands out the same blocks in the same order every `period` steps once it is warm (a
// step's allocations and releases are a fixed sequence), which makes the recorded pointers valid for every replay and
// leaves the host-side tensors pointing at the right blocks afterwards.  The period is measured, not assumed; without
// one the loop stays eager.  The step must do the same backend work every time it is called (no value read back from
// the device may steer it) and may not keep tensors it creates from one call to the next, other than through the
// tensors it updates (parameters, gradients).  Returns the number of steps that were replays.
template <class B, class Step>
size_t run_steps(Step&& step, size_t epochs, bool allow_graph) {
    size_t done = 0, replayed = 0;
    // MXT_TRACE_STEPS in the environment: where the wall-clock time of a call goes (warm-up, recording, replays, the rest)
    static const bool trace_steps = std::getenv("MXT_TRACE_STEPS") != nullptr;
    const auto clock0 = std::chrono::steady_clock::now();
    auto since = [&] { return std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - clock0).count(); };
    if constexpr (B::has_graphs) {
        constexpr size_t kMinWarm = 8, kMaxWarm = 64, kMaxPeriod = 4;   // the README loop settles into period 3 after 5 steps
        if (allow_graph && epochs >= 4 * kMinWarm) {
            Pool<B>& pool = Pool<B>::instance();
            std::vector<std::vector<void*>> traces;
            size_t period = 0;
            const size_t warm_limit = std::min<size_t>(kMaxWarm, epochs / 2);
            while (done < warm_limit && !period) {
                traces.emplace_back();
                pool.trace = &traces.back();
                step(done);
                pool.trace = nullptr;
                ++done;
                const size_t n = traces.size();
                if (n < kMinWarm) continue;
                // a period p is accepted when the last 2p steps repeat the p steps before them
                for (size_t p = 1; p <= kMaxPeriod && !period && 3 * p <= n; ++p) {
                    bool same = true;
                    for (size_t k = 0; k < 2 * p && same; ++k) same = traces[n - 1 - k] == traces[n - 1 - k - p];
                    if (same) period = p;
                }
            }
            if (trace_steps) std::fprintf(stderr, "run_steps: %zu eager steps until period %zu: %.3f ms\n", done, period, since());
            if (period) {
                const size_t one = period, warm = traces.size();
                // Records `span` steps (a multiple of the period) and replays them as often as whole spans fit; false when
                // the recording left the allocation pattern (it then ran once, and the loop goes on eagerly).  The recorded
                // steps must follow the pattern the warm-up settled into: a replay runs on the addresses recorded, and is
                // only the next step's work if that step would have used the same ones.
                auto record_and_replay = [&](size_t span) {
                    void* exec = nullptr;
                    const size_t allocs_before = pool.device_allocs, calls_before = backend_calls();
                    std::vector<std::vector<void*>> recorded(span);
                    B::graph_begin();
                    try {
                        for (size_t k = 0; k < span; ++k) {
                            pool.trace = &recorded[k];
                            step(done + k);
                            pool.trace = nullptr;
                        }
                    } catch (...) {
                        pool.trace = nullptr;
                        try { B::graph_end(&exec); } catch (...) { exec = nullptr; }
                        if (exec) B::graph_destroy(exec);
                        throw;
                    }
                    if (trace_steps) std::fprintf(stderr, "run_steps: %zu steps recorded: %.3f ms\n", span, since());
                    B::graph_end(&exec);
                    if (trace_steps) std::fprintf(stderr, "run_steps: recording closed: %.3f ms\n", since());
                    bool periodic = true;
                    for (size_t k = 0; k < span && periodic; ++k) periodic = recorded[k] == traces[warm - one + k % one];
                    if (pool.device_allocs != allocs_before) {
                        B::graph_destroy(exec);
                        throw Error(ErrKind::Backend, "the step allocated device memory while it was being recorded");
                    }
                    // the recorded steps did not run yet: replay them, then as many more whole spans as fit
                    const size_t calls_per_span = backend_calls() - calls_before;
                    // (one call for all the replays: a backend that keeps the recording as a resident step program makes
                    // them in one launch)
                    size_t spans = periodic ? (epochs - done) / span : 1;
                    B::graph_launch_n(exec, spans);
                    if (trace_steps) std::fprintf(stderr, "run_steps: %zu replays of %zu steps queued: %.3f ms\n", spans, span, since());
                    backend_calls() += calls_per_span * (spans - 1);
                    done += spans * span;
                    replayed += spans * span;
                    B::graph_destroy(exec);
                    if (trace_steps) std::fprintf(stderr, "run_steps: recording released: %.3f ms\n", since());
                    return periodic;
                };
                // several periods per graph: a graph launch costs a few microseconds however many nodes it holds
                size_t span = one * std::max<size_t>(1, 12 / one);
                while (span > one && 2 * span > epochs - done) span -= one;
                record_and_replay(span);
            }
        }
    }
    const size_t rest = epochs - done;
    for (; done < epochs; ++done) step(done);
    if (trace_steps) std::fprintf(stderr, "run_steps: %zu eager steps at the end, all queued: %.3f ms\n", rest, since());
    return replayed;
}

// ---- the training loop of examples/device/cpu.rs:32-38 -----------------------------------------------
// forward, loss, backward, optimizer step, zero_grad.  `losses` (may be null) receives every epoch's loss, which
// costs a device-to-host copy per epoch (and keeps the loop eager: see run_steps).
template <class B, class Model>
size_t train_loop(Model& model, const Tensor<B>& x, const Tensor<B>& y, float lr, size_t epochs, float* losses, bool allow_graph) {
    SGD<B> opt(lr);
    auto step = [&](size_t e) {
        Tensor<B> pred = model.forward(x);
        Tensor<B> loss = mse_loss<B>(pred, y);
        loss.backward();
        opt.step(model.parameters());
        opt.zero_grad(model.parameters());
        if (losses) losses[e] = loss.item();
    };
    return run_steps<B>(step, epochs, allow_graph && !losses);
}

}  // namespace mxt
