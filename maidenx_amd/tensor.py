"""Python face of the host layer (libmaidenx_host.so, C ABI in include/maidenx_host.h).

    from maidenx_amd.tensor import host
    mx = host()                      # the HIP-backed library; raises if it is not built
    x = mx.tensor([[1., 2.], [3., 4.]]).with_grad()
    y = x.mul(x).sum_all(); y.backward(); x.grad().numpy()

Method names follow crates/maidenx_tensor (add, sub, mul, div, matmul, sum, sum_to_shape, transpose,
reshape, ...) and crates/maidenx_nn (Linear, Conv2d, MSELoss, SGD).  Errors of the reference's `Result`
become `MxError` with the variant name in `.kind`.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
HOST_LIB_PATH = os.path.join(_HERE, "libmaidenx_host.so")

DTYPES = ["f32", "bf16", "bool"]
_KINDS = ["None", "InvalidShape", "ShapeMismatch", "DimensionOutOfBounds", "IncompatibleShape", "InvalidOperation",
          "InvalidArgument", "UnsupportedDType", "OutOfMemory", "Backend"]


STEP_FN = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_size_t)      # mxt_step_fn


class MxError(RuntimeError):
    def __init__(self, kind, text):
        super().__init__(f"{kind}: {text}")
        self.kind = kind


def _bind(lib):
    P, SZ, I, F = C.c_void_p, C.c_size_t, C.c_int, C.c_float
    sig = {
        "mxt_last_error": ([C.c_char_p, SZ], I), "mxt_backend_name": ([], C.c_char_p),
        "mxt_new": ([P, P, SZ], P), "mxt_fill": ([P, SZ, F], P), "mxt_new_dtype": ([P, P, SZ, I], P), "mxt_fill_dtype": ([P, SZ, F, I], P),
        "mxt_dtype": ([P], I), "mxt_to_dtype": ([P, I], P), "mxt_cast_calls": ([], SZ), "mxt_randn": ([P, SZ, C.c_uint64], P), "mxt_release": ([P], None),
        "mxt_ndim": ([P], SZ), "mxt_size": ([P], SZ), "mxt_offset": ([P], SZ), "mxt_shape": ([P, P], None), "mxt_strides": ([P, P], None),
        "mxt_requires_grad": ([P], I), "mxt_is_contiguous": ([P], I), "mxt_to_host": ([P, P], I),
        "mxt_with_grad": ([P], I), "mxt_grad": ([P], P), "mxt_backward": ([P], I), "mxt_zero_grad": ([P], I), "mxt_detach": ([P], P),
        "mxt_binary": ([C.c_char_p, P, P], P), "mxt_binary_inplace": ([C.c_char_p, P, P], I), "mxt_unary": ([C.c_char_p, P], P),
        "mxt_unary_scalar": ([C.c_char_p, P, F], P), "mxt_reduce": ([C.c_char_p, P, I, I], P), "mxt_shape_op": ([C.c_char_p, P, P, SZ], P),
        "mxt_linear_new": ([P, P], P), "mxt_linear_new_seeded": ([SZ, SZ, I, C.c_uint64], P),
        "mxt_conv2d_new": ([P, P, SZ, SZ, SZ, SZ, SZ, SZ], P), "mxt_module_forward": ([P, P], P), "mxt_module_weight": ([P], P),
        "mxt_module_bias": ([P], P), "mxt_module_release": ([P], None), "mxt_mse_loss": ([P, P], P), "mxt_sgd_step": ([P, F], I),
        "mxt_sgd_zero_grad": ([P], I), "mxt_train": ([P, P, P, F, SZ, P], I), "mxt_set_graph_replay": ([I], None),
        "mxt_last_train_replayed": ([], SZ), "mxt_run_steps": ([P, P, SZ], I), "mxt_set_conv_skip_unread_grad_cols": ([I], None), "mxt_set_autograd_shortcuts": ([I], None), "mxt_set_fused_nn_kernels": ([I], None), "mxt_set_sum_all_in_one_pass": ([I], None), "mxt_set_conv_gathered_products": ([I], None),
        "mxt_adam_new": ([C.c_double] * 4, P), "mxt_adam_release": ([P], None), "mxt_adam_set_fused": ([P, I], None), "mxt_adam_step": ([P, P], I),
        "mxt_backend_calls": ([], SZ), "mxt_reset_backend_calls": ([], None), "mxt_device_allocations": ([], SZ), "mxt_synchronize": ([], I),
    }
    for name, (args, res) in sig.items():
        fn = getattr(lib, name)
        fn.argtypes, fn.restype = args, res


class Host:
    """One loaded host-layer library (one backend)."""

    def __init__(self, path):
        if not os.path.exists(path):
            raise MxError("Backend", f"{path} is not built (python -m maidenx_amd.build)")
        self.lib = C.CDLL(path, mode=C.RTLD_GLOBAL)
        _bind(self.lib)
        self.name = self.lib.mxt_backend_name().decode()

    # -- error plumbing --
    def _raise(self):
        buf = C.create_string_buffer(1024)
        kind = self.lib.mxt_last_error(buf, 1024)
        raise MxError(_KINDS[kind] if 0 <= kind < len(_KINDS) else str(kind), buf.value.decode())

    def _t(self, handle):
        if not handle:
            self._raise()
        return Tensor(self, handle)

    def _rc(self, rc):
        if rc != 0:
            self._raise()

    # -- creation --
    def tensor(self, data, shape=None, dtype="f32"):
        """f32 values stored as `dtype` ("f32" or "bf16", rounded to nearest even)."""
        a = np.ascontiguousarray(data, dtype=np.float32)
        shp = tuple(a.shape if shape is None else shape)
        s = (C.c_size_t * max(1, len(shp)))(*shp)
        return self._t(self.lib.mxt_new_dtype(a.ctypes.data, s, len(shp), DTYPES.index(dtype)))

    def fill(self, shape, value, dtype="f32"):
        s = (C.c_size_t * max(1, len(shape)))(*shape)
        return self._t(self.lib.mxt_fill_dtype(s, len(shape), float(value), DTYPES.index(dtype)))

    def zeros(self, shape, dtype="f32"):
        return self.fill(shape, 0.0, dtype)

    def ones(self, shape, dtype="f32"):
        return self.fill(shape, 1.0, dtype)

    def randn(self, shape, seed):
        s = (C.c_size_t * max(1, len(shape)))(*shape)
        return self._t(self.lib.mxt_randn(s, len(shape), seed))

    # -- nn --
    def Linear(self, weight=None, bias=None, in_features=None, out_features=None, with_bias=True, seed=0):
        if weight is None:
            h = self.lib.mxt_linear_new_seeded(in_features, out_features, int(with_bias), seed)
        else:
            h = self.lib.mxt_linear_new(weight.h, bias.h if bias is not None else None)
        if not h:
            self._raise()
        return Module(self, h)

    def Conv2d(self, weight, bias=None, stride=(1, 1), padding=(0, 0)):
        kh, kw = weight.shape[2], weight.shape[3]
        h = self.lib.mxt_conv2d_new(weight.h, bias.h if bias is not None else None, kh, kw, stride[0], stride[1], padding[0], padding[1])
        if not h:
            self._raise()
        return Module(self, h)

    def Adam(self, lr=0.001, beta1=0.9, beta2=0.999, epsilon=1e-8):
        return Adam(self, lr, beta1, beta2, epsilon)

    def mse_loss(self, pred, target):
        return self._t(self.lib.mxt_mse_loss(pred.h, target.h))

    def train(self, module, x, y, lr, epochs, record_losses=False):
        """examples/device/cpu.rs:32-38, `epochs` times in native code."""
        losses = np.zeros(epochs, np.float32) if record_losses else None
        self._rc(self.lib.mxt_train(module.h, x.h, y.h, lr, epochs, losses.ctypes.data if record_losses else None))
        return losses

    def run_steps(self, step, n):
        """Runs step() n times, or - on the HIP build, from 32 steps on, once the buffer addresses of a step repeat - records
        it as a graph and replays that.  step() must issue the same tensor calls every time, read nothing back from the
        device and keep none of the tensors it creates; what it updates (parameters, gradients) is as after n calls."""
        failure = []

        def call(_user, _e):
            try:
                step()
                return 0
            except BaseException as ex:      # (must not travel through the native frames)
                failure.append(ex)
                return 1

        fn = STEP_FN(call)
        rc = self.lib.mxt_run_steps(C.cast(fn, C.c_void_p), None, n)
        if failure:
            raise failure[0]
        self._rc(rc)

    def set_graph_replay(self, enabled):
        self.lib.mxt_set_graph_replay(int(enabled))

    def last_train_replayed(self):
        return self.lib.mxt_last_train_replayed()

    def set_conv_skip_unread_grad_cols(self, enabled):
        """Conv2d backward computes only the rows of grad_cols that col2im reads (default), or the whole product."""
        self.lib.mxt_set_conv_skip_unread_grad_cols(int(enabled))

    def set_sum_all_in_one_pass(self, enabled):
        """sum_all() of a contiguous f32 tensor as one reduction (default) or dim by dim as the reference does."""
        self.lib.mxt_set_sum_all_in_one_pass(int(enabled))

    def set_autograd_shortcuts(self, enabled):
        """backward() skips work that cannot change any gradient (default), or does everything the reference does."""
        self.lib.mxt_set_autograd_shortcuts(int(enabled))

    def set_fused_nn_kernels(self, enabled):
        """MSELoss and SGD.step as one backend call each (default; same gradients and parameters bit for bit), or the op
        sequences of the reference."""
        self.lib.mxt_set_fused_nn_kernels(int(enabled))

    def set_conv_gathered_products(self, mode):
        """Conv2d's products with the column matrix: 0 = store the matrix first (im2col), 1 = gather it inside the product
        when no backward is recorded (default), 2 = gather always."""
        self.lib.mxt_set_conv_gathered_products(int(mode))

    def backend_calls(self):
        return self.lib.mxt_backend_calls()

    def cast_calls(self):
        return self.lib.mxt_cast_calls()

    def reset_backend_calls(self):
        self.lib.mxt_reset_backend_calls()

    def device_allocations(self):
        return self.lib.mxt_device_allocations()

    def synchronize(self):
        self._rc(self.lib.mxt_synchronize())


class Tensor:
    def __init__(self, host, handle):
        self.m, self.h = host, handle

    def __del__(self):
        try:
            self.m.lib.mxt_release(self.h)
        except Exception:
            pass

    # -- metadata --
    @property
    def shape(self):
        n = self.m.lib.mxt_ndim(self.h)
        out = (C.c_size_t * max(1, n))()
        self.m.lib.mxt_shape(self.h, out)
        return tuple(out[:n])

    @property
    def strides(self):
        n = self.m.lib.mxt_ndim(self.h)
        out = (C.c_size_t * max(1, n))()
        self.m.lib.mxt_strides(self.h, out)
        return tuple(out[:n])

    @property
    def dtype(self):
        return DTYPES[self.m.lib.mxt_dtype(self.h)]

    def to_dtype(self, dtype):
        return self.m._t(self.m.lib.mxt_to_dtype(self.h, DTYPES.index(dtype)))

    @property
    def offset(self):
        return self.m.lib.mxt_offset(self.h)

    @property
    def requires_grad(self):
        return bool(self.m.lib.mxt_requires_grad(self.h))

    def is_contiguous(self):
        return bool(self.m.lib.mxt_is_contiguous(self.h))

    def numpy(self):
        out = np.zeros(self.m.lib.mxt_size(self.h), np.float32)
        self.m._rc(self.m.lib.mxt_to_host(self.h, out.ctypes.data))
        return out.reshape(self.shape)

    def item(self):
        return float(self.numpy().reshape(-1)[0])

    # -- autograd --
    def with_grad(self):
        self.m._rc(self.m.lib.mxt_with_grad(self.h))
        return self

    def grad(self):
        h = self.m.lib.mxt_grad(self.h)
        return Tensor(self.m, h) if h else None

    def backward(self):
        self.m._rc(self.m.lib.mxt_backward(self.h))

    def zero_grad(self):
        self.m._rc(self.m.lib.mxt_zero_grad(self.h))

    def detach(self):
        return self.m._t(self.m.lib.mxt_detach(self.h))

    # -- ops --
    def _bin(self, op, other):
        return self.m._t(self.m.lib.mxt_binary(op, self.h, other.h))

    def _un(self, op):
        return self.m._t(self.m.lib.mxt_unary(op, self.h))

    def _unc(self, op, c):
        return self.m._t(self.m.lib.mxt_unary_scalar(op, self.h, float(c)))

    def _shp(self, op, args):
        a = (C.c_int64 * max(1, len(args)))(*[int(v) for v in args])
        return self.m._t(self.m.lib.mxt_shape_op(op, self.h, a, len(args)))

    def add(self, o): return self._bin(b"add", o)
    def sub(self, o): return self._bin(b"sub", o)
    def mul(self, o): return self._bin(b"mul", o)
    def div(self, o): return self._bin(b"div", o)
    def matmul(self, o): return self._bin(b"matmul", o)
    def add_(self, o): self.m._rc(self.m.lib.mxt_binary_inplace(b"add_", self.h, o.h))
    def sub_(self, o): self.m._rc(self.m.lib.mxt_binary_inplace(b"sub_", self.h, o.h))
    def neg(self): return self._un(b"neg")
    def square(self): return self._un(b"square")
    def relu(self): return self._un(b"relu")
    def tanh(self): return self._un(b"tanh")
    def gelu(self): return self._un(b"gelu")
    def exp(self): return self._un(b"exp")
    def sqrt(self): return self._un(b"sqrt")
    def sum_all(self): return self._un(b"sum_all")
    def mean_all(self): return self._un(b"mean_all")
    def contiguous(self): return self._un(b"contiguous")
    def squeeze_all(self): return self._un(b"squeeze_all")
    def add_scalar(self, c): return self._unc(b"add_scalar", c)
    def mul_scalar(self, c): return self._unc(b"mul_scalar", c)
    def div_scalar(self, c): return self._unc(b"div_scalar", c)
    def pow(self, c): return self._unc(b"pow", c)
    def gt_scalar(self, c): return self._unc(b"gt_scalar", c)
    def sum(self, dim, keep_dim=False): return self.m._t(self.m.lib.mxt_reduce(b"sum", self.h, dim, int(keep_dim)))
    def mean(self, dim, keep_dim=False): return self.m._t(self.m.lib.mxt_reduce(b"mean", self.h, dim, int(keep_dim)))
    def view(self, shape): return self._shp(b"view", shape)
    def reshape(self, shape): return self._shp(b"reshape", shape)
    def broadcast(self, shape): return self._shp(b"broadcast", shape)
    def broadcast_left(self, batch_dims): return self._shp(b"broadcast_left", batch_dims)
    def sum_to_shape(self, shape): return self._shp(b"sum_to_shape", shape)
    def transpose(self, d0, d1): return self._shp(b"transpose", (d0, d1))
    def squeeze(self, d): return self._shp(b"squeeze", (d,))
    def unsqueeze(self, d): return self._shp(b"unsqueeze", (d,))


class Module:
    def __init__(self, host, handle):
        self.m, self.h = host, handle

    def __del__(self):
        try:
            self.m.lib.mxt_module_release(self.h)
        except Exception:
            pass

    def forward(self, x):
        return self.m._t(self.m.lib.mxt_module_forward(self.h, x.h))

    @property
    def weight(self):
        return self.m._t(self.m.lib.mxt_module_weight(self.h))

    @property
    def bias(self):
        h = self.m.lib.mxt_module_bias(self.h)
        return Tensor(self.m, h) if h else None

    def sgd_step(self, lr):
        self.m._rc(self.m.lib.mxt_sgd_step(self.h, lr))

    def zero_grad(self):
        self.m._rc(self.m.lib.mxt_sgd_zero_grad(self.h))


class Adam:
    """crates/maidenx_nn/src/optimizers/adam.rs; the moments belong to this object."""

    def __init__(self, m, lr, beta1, beta2, epsilon):
        self.m = m
        self.h = m.lib.mxt_adam_new(lr, beta1, beta2, epsilon)

    def __del__(self):
        if getattr(self, "h", None):
            self.m.lib.mxt_adam_release(self.h)
            self.h = None

    def set_fused(self, enabled):
        self.m.lib.mxt_adam_set_fused(self.h, int(enabled))

    def step(self, module):
        self.m._rc(self.m.lib.mxt_adam_step(self.h, module.h))


_host = None


def host():
    """The HIP-backed host layer.  There is no CPU fallback: a missing library is an error."""
    global _host
    if _host is None:
        _host = Host(HOST_LIB_PATH)
    return _host
