"""Shared test plumbing: one `Runner` that calls either the CPU oracle (oracle/liboracle.so, host
arrays) or the HIP backend (maidenx_amd/libmaidenx_hip.so, device buffers) through the same C
argument lists, the metadata builders of the reference's tensor layer, bf16 helpers and error
measures."""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_LIB = os.path.join(ORACLE_DIR, "liboracle.so")

import maidenx_amd._signatures as S  # noqa: E402

NP = {"f32": np.float32, "bf16": np.uint16, "f16": np.uint16, "bool": np.uint8, "f64": np.float64, "i32": np.int32, "i64": np.int64,
      "u8": np.uint8, "u16": np.uint16, "u32": np.uint32, "u64": np.uint64, "i8": np.int8, "i16": np.int16}


# ---- bf16 <-> f32 on the host (round to nearest even, NaN quieted), as the `half` crate does ----
def f32_to_bf16(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    x = a.view(np.uint32).astype(np.uint64)
    nan = (x & 0x7FFFFFFF) > 0x7F800000
    r = (x + 0x7FFF + ((x >> 16) & 1)) >> 16
    r = np.where(nan, (x >> 16) | 0x40, r)
    return r.astype(np.uint16).reshape(a.shape)


def bf16_to_f32(b):
    b = np.ascontiguousarray(b, dtype=np.uint16)
    return (b.astype(np.uint32) << 16).view(np.float32).reshape(b.shape)


def to_storage(a, dt):
    """float values -> storage array of dtype tag dt."""
    if dt == "bf16":
        return f32_to_bf16(np.asarray(a, dtype=np.float32))
    if dt == "f16":      # numpy's float16 is IEEE binary16 with round-to-nearest-even conversions
        with np.errstate(over="ignore"):
            return np.ascontiguousarray(np.asarray(a, dtype=np.float32).astype(np.float16)).view(np.uint16)
    return np.ascontiguousarray(a, dtype=NP[dt])


def to_float(a, dt):
    if dt == "bf16":
        return bf16_to_f32(a)
    if dt == "f16":
        return np.ascontiguousarray(a, dtype=np.uint16).view(np.float16).astype(np.float32)
    return np.asarray(a)


def ulp_diff_f32(a, b):
    """Distance in units in the last place between two f32 arrays (NaN==NaN, +0==-0)."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    ia = a.view(np.int32).astype(np.int64)
    ib = b.view(np.int32).astype(np.int64)
    ia = np.where(ia < 0, -(ia & 0x7FFFFFFF), ia)
    ib = np.where(ib < 0, -(ib & 0x7FFFFFFF), ib)
    d = np.abs(ia - ib)
    both_nan = np.isnan(a) & np.isnan(b)
    return np.where(both_nan, 0, d)


# ---- metadata builders (layouts of crates/maidenx_tensor/src/ops/*.rs) -----------------------------
def u64(*parts):
    out = []
    for p in parts:
        if np.isscalar(p):
            out.append(int(p))
        else:
            out.extend(int(v) for v in p)
    return np.array(out, dtype=np.uint64)


def contiguous_strides(dims):
    s, acc = [], 1
    for d in reversed(dims):
        s.append(acc)
        acc *= d
    return list(reversed(s))


def meta_binary(dims, ls, rs, lo=0, ro=0):      # tensor/ops/binary.rs:754-769
    return u64(dims, ls, rs, lo, ro)


def meta_unary(dims, strides, off=0):           # tensor/ops/unary.rs:1309-1320
    return u64(dims, strides, off)


def meta_reduce(dims, strides, dim, off=0):     # tensor/ops/reduction.rs:722-732 (one reduced dim)
    return u64(dims, strides, dims[dim], strides[dim], off)


def meta_sum_to_shape(dims, strides, out_dims, off=0):   # tensor/ops/reduction.rs:734-743
    return u64(dims, strides, out_dims, off)


def meta_matmul(out_shape, a_shape, b_shape, a_strides, b_strides, a_off=0, b_off=0):   # tensor/ops/matmul.rs:227-264
    return u64(len(out_shape), len(a_shape), len(b_shape), out_shape, a_shape, b_shape, a_strides, b_strides, a_off, b_off)


def meta_pad(in_dims, in_strides, in_off, out_dims, pads):   # tensor/ops/padding.rs:272-294
    flat = [v for p in pads for v in p]
    return u64(in_dims, in_strides, in_off, out_dims, flat)


def layout(dims, strides=None, off=0):
    """dims[n] | strides[n] | offset of one tensor, as the index ops take it."""
    return u64(dims, strides if strides is not None else contiguous_strides(dims), off)


def meta_conv(B, Cc, H, W, kh, kw, oh, ow, pad_h, pad_w, stride_h, stride_w):
    """12 slots in the order the kernels READ them (maidenx_cpu nn/conv.rs:20-34)."""
    return u64(B, Cc, H, W, kh, kw, oh, ow, pad_h, pad_w, stride_h, stride_w)


# ---- argument wrappers -------------------------------------------------------------------------------
class In:
    def __init__(self, arr):
        self.arr = np.ascontiguousarray(arr)


class Out:
    """Output buffer of `count` elements; pre-filled with a poison pattern to catch partial writes."""

    def __init__(self, count, dt):
        self.dt = dt
        self.arr = np.empty(int(count), dtype=NP[dt])
        self.arr.view(np.uint8)[:] = 0xCD if dt != "bool" else 0x7


class InOut(In):
    pass


class Null:
    pass


ORACLE_HOST_LIB = os.path.join(ORACLE_DIR, "liboracle_host.so")


def ensure_oracle_built():
    if not os.path.exists(ORACLE_LIB) or not os.path.exists(ORACLE_HOST_LIB):
        subprocess.run(["make", "-C", ORACLE_DIR, "-j8", "all"], check=True, capture_output=True)
    return ORACLE_LIB


def oracle_host():
    """The product's host layer (tensor / autograd / nn) instantiated over the CPU oracle."""
    from maidenx_amd.tensor import Host
    ensure_oracle_built()
    return Host(ORACLE_HOST_LIB)


class Runner:
    """kind = 'oracle' (CPU restatement, test infrastructure) or 'hip' (the product, on the GPU)."""

    def __init__(self, kind):
        self.kind = kind
        if kind == "oracle":
            self.lib = C.CDLL(ensure_oracle_built())
            self.prefix = "oracle_"
            for name, args in {**S.signatures(("f32", "bf16", "f16", "f64")), **S.binary_signatures(), **S.index_signatures()}.items():
                fn = getattr(self.lib, self.prefix + name)
                fn.argtypes = args
                fn.restype = None
            for name, args in {**S.cast_signatures(), **S.wide_unary_signatures(tuple(d for d in S.WIDE_DTYPES if d != "f64")),
                               **S.wide_reduce_signatures(tuple(d for d in S.REDUCE_WIDE_DTYPES if d != "f64"))}.items():
                fn = getattr(self.lib, self.prefix + name)
                fn.argtypes = args
                fn.restype = None
            self.lib.oracle_index_error.restype = C.c_int
            self.lib.oracle_set_num_threads.argtypes = [C.c_int]
            self.lib.oracle_set_num_threads.restype = C.c_int
        else:
            import maidenx_amd.lib as L
            self.L = L
            self.lib = L.load()
            self.prefix = "hip_"

    def set_threads(self, n):
        assert self.kind == "oracle"
        return self.lib.oracle_set_num_threads(int(n))

    def call(self, name, *args):
        fn = getattr(self.lib, self.prefix + name)
        cargs, post = [], []
        keep = []
        seen = {}
        for a in args:
            if isinstance(a, Null) or a is None:
                cargs.append(None)
            elif isinstance(a, (In, Out)):
                if self.kind == "oracle":
                    cargs.append(a.arr.ctypes.data)
                elif id(a) in seen:                      # the same In object given twice: one buffer, the same pointer
                    cargs.append(seen[id(a)].ptr)
                else:
                    buf = self.L.DeviceBuffer.from_numpy(a.arr)
                    seen[id(a)] = buf
                    keep.append(buf)
                    cargs.append(buf.ptr)
                    if isinstance(a, (Out, InOut)):
                        post.append((a, buf))
            elif isinstance(a, np.ndarray):      # host metadata
                keep.append(a)
                cargs.append(a.ctypes.data)
            else:
                cargs.append(a)
        self.last_return = fn(*cargs)        # (None for the void entry points)
        if self.kind == "hip":
            for a, buf in post:
                a.arr[...] = buf.to_numpy(a.arr.dtype, a.arr.size)
            self.L.synchronize()
        return [a.arr for a in args if isinstance(a, (Out, InOut))]


def const_arg(v, dt):
    """A by-value constant of the input dtype."""
    if dt in ("bf16", "f16"):
        return int(to_storage(np.array([v], dtype=np.float32), dt)[0])
    if dt in ("f32", "f64"):
        return float(v)
    return int(v)


def rng(seed):
    return np.random.default_rng(seed)


PLAIN = ["f32", "f64", "bool", "u8", "u16", "u32", "u64", "i8", "i16", "i32", "i64"]


def cast_inputs(dt, n=3000, seed=21):
    """Source values for the dtype conversions: every boundary of every integer target, just inside and just outside,
    fractions either side of zero, NaN and infinities for the floats; extremes and random fill for the integers."""
    r = rng(seed)
    if dt in ("f32", "f64"):
        ft = NP[dt]
        edges = []
        for bits in (8, 16, 32, 64):
            for v in (2.0 ** bits, 2.0 ** (bits - 1), -(2.0 ** (bits - 1))):
                x = ft(v)
                edges += [x, np.nextafter(x, ft(np.inf)), np.nextafter(x, ft(-np.inf)), x + ft(0.5), x - ft(0.5), x - ft(1), x + ft(1)]
        edges += [0.0, -0.0, 0.5, -0.5, 0.999, -0.999, 1.5, -1.5, 255.5, -128.5, np.nan, np.inf, -np.inf, 1e30, -1e30, 3e38]
        scale = r.choice([1.0, 1e2, 1e5, 1e10, 1e19], n - len(edges))
        with np.errstate(over="ignore"):
            x = np.concatenate([np.array(edges, dtype=ft), (r.standard_normal(n - len(edges)) * scale).astype(ft)])
        return x
    if dt == "bool":
        return r.integers(0, 2, n, dtype=np.uint8)
    info = np.iinfo(NP[dt])
    x = r.integers(info.min, info.max, n, dtype=NP[dt], endpoint=True)
    x[: n // 3] = r.integers(max(info.min, -300), min(info.max, 300), n // 3, dtype=NP[dt], endpoint=True)
    edge = [info.min, info.max, 0, 1, info.max - 1, info.min + 1, info.max // 2, info.max // 2 + 1]
    for bits in (8, 16, 24, 25, 32, 53, 54, 63):           # where narrower integers wrap and floats start to round
        for v in (2 ** bits - 1, 2 ** bits, 2 ** bits + 1, 2 ** bits + 3):
            if v <= info.max:
                edge.append(v)
            if -v >= info.min:
                edge.append(-v)
    x[-len(edge):] = np.array(edge, dtype=object).astype(NP[dt])
    return x
