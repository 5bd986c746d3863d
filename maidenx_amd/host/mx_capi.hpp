// The C ABI of the host layer (include/maidenx_host.h) for one backend.  Include after defining the
// backend struct and `using MxtBackend = ...;`.
#pragma once
#include <cstdio>

#include "../../include/maidenx_host.h"
#include "mx_tensor.hpp"

namespace mxt_capi {
using B = MxtBackend;
using T = mxt::Tensor<B>;

struct Module {
    int kind;                                     // 0 linear, 1 conv2d
    std::unique_ptr<mxt::Linear<B>> linear;
    std::unique_ptr<mxt::Conv2d<B>> conv;
    std::vector<T*> parameters() { return kind == 0 ? linear->parameters() : conv->parameters(); }
    T forward(const T& x) const { return kind == 0 ? linear->forward(x) : conv->forward(x); }
};

inline bool g_graphs = true;
inline size_t g_replayed = 0;
inline thread_local int g_kind = 0;
inline thread_local std::string g_text;
inline void set_error(int k, const std::string& t) { g_kind = k; g_text = t; }

template <class F>
mxt_tensor guard_t(F&& f) {
    try {
        return new T(f());
    } catch (const mxt::Error& e) {
        set_error((int)e.kind, e.what());
    } catch (const std::exception& e) {
        set_error(MXT_ERR_BACKEND, e.what());
    }
    return nullptr;
}
template <class F>
int guard_i(F&& f) {
    try {
        f();
        return 0;
    } catch (const mxt::Error& e) {
        set_error((int)e.kind, e.what());
        return (int)e.kind;
    } catch (const std::exception& e) {
        set_error(MXT_ERR_BACKEND, e.what());
        return MXT_ERR_BACKEND;
    }
}
inline T& ref(mxt_tensor t) {
    if (!t) throw mxt::Error(mxt::ErrKind::InvalidArgument, "null tensor handle");
    return *(T*)t;
}
inline mxt::Shape to_shape(const size_t* s, size_t n) { return mxt::Shape(s, s + n); }
inline bool is(const char* a, const char* b) { return std::strcmp(a, b) == 0; }
[[noreturn]] inline void unknown(const char* family, const char* op) {
    throw mxt::Error(mxt::ErrKind::InvalidArgument, std::string("unknown ") + family + " op '" + op + "'");
}
}  // namespace mxt_capi

extern "C" {
using namespace mxt_capi;

int mxt_last_error(char* text, size_t cap) {
    if (text && cap) std::snprintf(text, cap, "%s", g_text.c_str());
    return g_kind;
}
const char* mxt_backend_name(void) { return B::name; }

mxt_tensor mxt_new(const float* data, const size_t* shape, size_t ndim) {
    return guard_t([&] { return T::from_host(data, to_shape(shape, ndim)); });
}
mxt_tensor mxt_fill(const size_t* shape, size_t ndim, float value) {
    return guard_t([&] { return T::fill(to_shape(shape, ndim), value); });
}
static mxt::DType dtype_of(int code) {
    if (code == MXT_F32) return mxt::DType::F32;
    if (code == MXT_BF16) return mxt::DType::BF16;
    if (code == MXT_BOOL) return mxt::DType::BOOL;
    throw mxt::Error(mxt::ErrKind::InvalidArgument, "unknown dtype code");
}
mxt_tensor mxt_new_dtype(const float* data, const size_t* shape, size_t ndim, int dtype) {
    return guard_t([&] { return T::from_host(data, to_shape(shape, ndim), dtype_of(dtype)); });
}
mxt_tensor mxt_fill_dtype(const size_t* shape, size_t ndim, float value, int dtype) {
    return guard_t([&] { return T::fill(to_shape(shape, ndim), value, dtype_of(dtype)); });
}
mxt_tensor mxt_randn(const size_t* shape, size_t ndim, uint64_t seed) {
    return guard_t([&] { return mxt::randn<B>(to_shape(shape, ndim), seed); });
}
void mxt_release(mxt_tensor t) { delete (T*)t; }

size_t mxt_ndim(mxt_tensor t) { return ((T*)t)->ndim(); }
size_t mxt_size(mxt_tensor t) { return ((T*)t)->size(); }
size_t mxt_offset(mxt_tensor t) { return ((T*)t)->offset(); }
void mxt_shape(mxt_tensor t, size_t* out) { for (size_t i = 0; i < ((T*)t)->ndim(); ++i) out[i] = ((T*)t)->shape()[i]; }
void mxt_strides(mxt_tensor t, size_t* out) { for (size_t i = 0; i < ((T*)t)->ndim(); ++i) out[i] = ((T*)t)->strides()[i]; }
int mxt_dtype(mxt_tensor t) {
    mxt::DType d = ((T*)t)->dtype;
    return d == mxt::DType::F32 ? MXT_F32 : d == mxt::DType::BF16 ? MXT_BF16 : MXT_BOOL;
}
mxt_tensor mxt_to_dtype(mxt_tensor t, int dtype) { return guard_t([&] { return ref(t).to_dtype(dtype_of(dtype)); }); }
int mxt_requires_grad(mxt_tensor t) { return ((T*)t)->requires_grad ? 1 : 0; }
int mxt_is_contiguous(mxt_tensor t) { return ((T*)t)->is_contiguous() ? 1 : 0; }
int mxt_to_host(mxt_tensor t, float* out) {
    return guard_i([&] {
        std::vector<float> v = ref(t).to_vec();
        if (!v.empty()) std::memcpy(out, v.data(), v.size() * sizeof(float));
    });
}

int mxt_with_grad(mxt_tensor t) { return guard_i([&] { ref(t).with_grad(); }); }
mxt_tensor mxt_grad(mxt_tensor t) {
    if (!t || !((T*)t)->has_grad()) return nullptr;
    return guard_t([&] { return ref(t).grad(); });
}
int mxt_backward(mxt_tensor t) { return guard_i([&] { ref(t).backward(); }); }
int mxt_zero_grad(mxt_tensor t) { return guard_i([&] { ref(t).zero_grad(); }); }
mxt_tensor mxt_detach(mxt_tensor t) { return guard_t([&] { return ref(t).detach(); }); }

mxt_tensor mxt_binary(const char* op, mxt_tensor a, mxt_tensor b) {
    return guard_t([&]() -> T {
        T &x = ref(a), &y = ref(b);
        if (is(op, "add")) return x.add(y);
        if (is(op, "sub")) return x.sub(y);
        if (is(op, "mul")) return x.mul(y);
        if (is(op, "div")) return x.div(y);
        if (is(op, "matmul")) return x.matmul(y);
        unknown("binary", op);
    });
}
int mxt_binary_inplace(const char* op, mxt_tensor a, mxt_tensor b) {
    return guard_i([&] {
        T &x = ref(a), &y = ref(b);
        if (is(op, "add_")) x.add_(y);
        else if (is(op, "sub_")) x.sub_(y);
        else unknown("in-place", op);
    });
}
mxt_tensor mxt_unary(const char* op, mxt_tensor a) {
    return guard_t([&]() -> T {
        T& x = ref(a);
        if (is(op, "neg")) return x.neg();
        if (is(op, "sqrt")) return x.sqrt();
        if (is(op, "square")) return x.square();
        if (is(op, "relu")) return x.relu();
        if (is(op, "tanh")) return x.tanh();
        if (is(op, "gelu")) return x.gelu();
        if (is(op, "exp")) return x.exp();
        if (is(op, "sum_all")) return x.sum_all();
        if (is(op, "mean_all")) return x.mean_all();
        if (is(op, "contiguous")) return x.contiguous();
        if (is(op, "squeeze_all")) return x.squeeze_all();
        unknown("unary", op);
    });
}
mxt_tensor mxt_unary_scalar(const char* op, mxt_tensor a, float c) {
    return guard_t([&]() -> T {
        T& x = ref(a);
        if (is(op, "add_scalar")) return x.add_scalar(c);
        if (is(op, "mul_scalar")) return x.mul_scalar(c);
        if (is(op, "div_scalar")) return x.div_scalar(c);
        if (is(op, "pow")) return x.pow(c);
        if (is(op, "gt_scalar")) return x.gt_scalar(c);
        unknown("scalar", op);
    });
}
mxt_tensor mxt_reduce(const char* op, mxt_tensor a, int dim, int keep_dim) {
    return guard_t([&]() -> T {
        T& x = ref(a);
        if (is(op, "sum")) return x.sum(dim, keep_dim != 0);
        if (is(op, "mean")) return x.mean(dim, keep_dim != 0);
        unknown("reduce", op);
    });
}
mxt_tensor mxt_shape_op(const char* op, mxt_tensor a, const int64_t* args, size_t nargs) {
    return guard_t([&]() -> T {
        T& x = ref(a);
        std::vector<long> v(args, args + nargs);
        auto as_shape = [&] {
            mxt::Shape s;
            for (long d : v) {
                if (d < 0) throw mxt::Error(mxt::ErrKind::InvalidShape, "negative dimension");
                s.push_back((size_t)d);
            }
            return s;
        };
        if (is(op, "view")) return x.view(v);
        if (is(op, "reshape")) return x.reshape(v);
        if (is(op, "broadcast")) return x.broadcast(as_shape());
        if (is(op, "broadcast_left")) return x.broadcast_left(as_shape());
        if (is(op, "sum_to_shape")) return x.sum_to_shape(as_shape());
        if (is(op, "transpose") && nargs == 2) return x.transpose((int)v[0], (int)v[1]);
        if (is(op, "squeeze") && nargs == 1) return x.squeeze((int)v[0]);
        if (is(op, "unsqueeze") && nargs == 1) return x.unsqueeze((int)v[0]);
        unknown("shape", op);
    });
}

mxt_module mxt_linear_new(mxt_tensor weight, mxt_tensor bias) {
    Module* m = nullptr;
    int rc = guard_i([&] {
        auto mod = std::make_unique<Module>();
        mod->kind = 0;
        mod->linear = std::make_unique<mxt::Linear<B>>(ref(weight), bias ? (T*)bias : nullptr);
        m = mod.release();
    });
    return rc ? nullptr : m;
}
mxt_module mxt_linear_new_seeded(size_t in_features, size_t out_features, int with_bias, uint64_t seed) {
    Module* m = nullptr;
    int rc = guard_i([&] {
        auto mod = std::make_unique<Module>();
        mod->kind = 0;
        mod->linear = std::make_unique<mxt::Linear<B>>(in_features, out_features, with_bias != 0, seed);
        m = mod.release();
    });
    return rc ? nullptr : m;
}
mxt_module mxt_conv2d_new(mxt_tensor weight, mxt_tensor bias, size_t kh, size_t kw, size_t stride_h, size_t stride_w,
                          size_t pad_h, size_t pad_w) {
    Module* m = nullptr;
    int rc = guard_i([&] {
        if (ref(weight).ndim() != 4) throw mxt::Error(mxt::ErrKind::InvalidShape, "conv2d weight must be [Cout, Cin, kh, kw]");
        if (stride_h == 0 || stride_w == 0) throw mxt::Error(mxt::ErrKind::InvalidArgument, "conv2d stride must be positive");
        auto mod = std::make_unique<Module>();
        mod->kind = 1;
        mod->conv = std::make_unique<mxt::Conv2d<B>>(ref(weight), bias ? (T*)bias : nullptr, kh, kw, stride_h, stride_w, pad_h, pad_w);
        m = mod.release();
    });
    return rc ? nullptr : m;
}
mxt_tensor mxt_module_forward(mxt_module m, mxt_tensor input) {
    return guard_t([&] { return ((Module*)m)->forward(ref(input)); });
}
mxt_tensor mxt_module_weight(mxt_module m) { return guard_t([&] { return *((Module*)m)->parameters()[0]; }); }
mxt_tensor mxt_module_bias(mxt_module m) {
    auto p = ((Module*)m)->parameters();
    if (p.size() < 2) return nullptr;
    return guard_t([&] { return *p[1]; });
}
void mxt_module_release(mxt_module m) { delete (Module*)m; }
mxt_tensor mxt_mse_loss(mxt_tensor pred, mxt_tensor target) {
    return guard_t([&] { return mxt::mse_loss<B>(ref(pred), ref(target)); });
}
int mxt_sgd_step(mxt_module m, float lr) { return guard_i([&] { mxt::SGD<B>(lr).step(((Module*)m)->parameters()); }); }
int mxt_sgd_zero_grad(mxt_module m) { return guard_i([&] { mxt::SGD<B>(0.0f).zero_grad(((Module*)m)->parameters()); }); }

void* mxt_adam_new(double lr, double beta1, double beta2, double epsilon) { return new mxt::Adam<B>(lr, beta1, beta2, epsilon); }
void mxt_adam_release(void* opt) { delete (mxt::Adam<B>*)opt; }
void mxt_adam_set_fused(void* opt, int enabled) { ((mxt::Adam<B>*)opt)->fused = enabled != 0; }
int mxt_adam_step(void* opt, mxt_module m) { return guard_i([&] { ((mxt::Adam<B>*)opt)->step(((Module*)m)->parameters()); }); }

int mxt_train(mxt_module m, mxt_tensor input, mxt_tensor target, float lr, size_t epochs, float* losses) {
    return guard_i([&] { g_replayed = mxt::train_loop<B>(*(Module*)m, ref(input), ref(target), lr, epochs, losses, g_graphs); });
}
int mxt_run_steps(mxt_step_fn fn, void* user, size_t steps) {
    return guard_i([&] {
        if (!fn) throw mxt::Error(mxt::ErrKind::InvalidArgument, "run_steps: no step function");
        g_replayed = mxt::run_steps<B>([&](size_t e) {
            if (fn(user, e) != 0) throw mxt::Error(mxt::ErrKind::InvalidOperation, "run_steps: the step function reported a failure");
        }, steps, g_graphs);
    });
}
void mxt_set_graph_replay(int enabled) { g_graphs = enabled != 0; }
size_t mxt_last_train_replayed(void) { return g_replayed; }
void mxt_set_sum_all_in_one_pass(int enabled) { mxt::sum_all_in_one_pass() = enabled != 0; }
void mxt_set_autograd_shortcuts(int enabled) { mxt::autograd_shortcuts() = enabled != 0; }
void mxt_set_fused_nn_kernels(int enabled) { mxt::fused_nn_kernels() = enabled != 0; }
void mxt_set_conv_skip_unread_grad_cols(int enabled) { mxt::conv_skip_unread_grad_cols() = enabled != 0; }
void mxt_set_conv_gathered_products(int mode) { mxt::conv_gathered_products() = mode < 0 ? 0 : mode > 2 ? 2 : mode; }

size_t mxt_backend_calls(void) { return mxt::backend_calls(); }
void mxt_reset_backend_calls(void) { mxt::backend_calls() = 0; mxt::cast_calls() = 0; }
size_t mxt_cast_calls(void) { return mxt::cast_calls(); }
size_t mxt_device_allocations(void) { return mxt::Pool<B>::instance().device_allocs; }
int mxt_synchronize(void) { return guard_i([&] { B::sync(); B::check(); }); }
}  // extern "C"
