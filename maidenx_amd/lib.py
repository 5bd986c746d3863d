"""ctypes binding of libmaidenx_hip.so — the C ABI declared in include/maidenx_hip.h.

Loading fails loudly when the library has not been built; there is no CPU fallback of any kind.
"""
import ctypes as C
import os

import numpy as np

from . import _signatures as S

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmaidenx_hip.so")

_lib = None


class HipError(RuntimeError):
    pass


def load():
    """Return the loaded library, binding argument types on first use."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise HipError(f"{LIB_PATH} is missing: build it with `python -m maidenx_amd.build` (needs hipcc)")
    lib = C.CDLL(LIB_PATH)
    for name, args in {**S.signatures(), **S.binary_signatures(), **S.extension_signatures()}.items():
        fn = getattr(lib, "hip_" + name)
        fn.argtypes = args
        fn.restype = None
    for name, args, res in [
        ("hip_get_last_status", [], C.c_int), ("hip_status_string", [], C.c_char_p),
        ("hip_set_device", [C.c_int], C.c_int), ("hip_get_device", [C.POINTER(C.c_int)], C.c_int),
        ("hip_device_count", [C.POINTER(C.c_int)], C.c_int),
        ("hip_malloc", [C.POINTER(C.c_void_p), C.c_size_t], C.c_int), ("hip_free", [C.c_void_p], C.c_int),
        ("hip_memcpy_h2d", [C.c_void_p, C.c_void_p, C.c_size_t], C.c_int),
        ("hip_memcpy_d2h", [C.c_void_p, C.c_void_p, C.c_size_t], C.c_int),
        ("hip_memcpy_d2d", [C.c_void_p, C.c_void_p, C.c_size_t], C.c_int),
        ("hip_stream_create", [C.POINTER(C.c_void_p)], C.c_int), ("hip_stream_destroy", [C.c_void_p], C.c_int),
        ("hip_stream_synchronize", [C.c_void_p], C.c_int), ("hip_set_stream", [C.c_void_p], C.c_int),
        ("hip_get_stream", [], C.c_void_p), ("hip_synchronize", [], C.c_int),
        ("hip_event_create", [C.POINTER(C.c_void_p)], C.c_int), ("hip_event_destroy", [C.c_void_p], C.c_int),
        ("hip_event_record", [C.c_void_p], C.c_int), ("hip_event_synchronize", [C.c_void_p], C.c_int),
        ("hip_event_elapsed_ms", [C.c_void_p, C.c_void_p, C.POINTER(C.c_float)], C.c_int),
        ("hip_graph_begin_capture", [], C.c_int), ("hip_graph_end_capture", [C.POINTER(C.c_void_p)], C.c_int),
        ("hip_graph_launch", [C.c_void_p], C.c_int), ("hip_graph_destroy", [C.c_void_p], C.c_int),
        ("hip_graph_is_program", [C.c_void_p], C.c_int), ("hip_graph_set_programs", [C.c_int], C.c_int),
        ("hip_graph_fused_launches", [C.c_void_p, C.POINTER(C.c_int)], C.c_int), ("hip_graph_set_fusion", [C.c_int], C.c_int),
        ("hip_noalloc_prepare", [], C.c_int), ("hip_scratch_allocations", [], C.c_size_t),
        ("hip_graph_launch_n", [C.c_void_p, C.c_size_t], C.c_int),
        ("hip_graph_is_resident", [C.c_void_p, C.POINTER(C.c_int), C.POINTER(C.c_int)], C.c_int),
        ("hip_graph_set_resident", [C.c_int], C.c_int), ("hip_buffer_discard", [C.c_void_p, C.c_size_t], None),
        ("hip_conv2d_forward_product_f32", [C.c_size_t] * 4 + [C.c_void_p] * 4, C.c_int),
    ]:
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = res
    _lib = lib
    return lib


def device_count():
    n = C.c_int(0)
    rc = load().hip_device_count(C.byref(n))
    return n.value if rc == 0 else 0


def check():
    """Raise if any call since the last check recorded an error."""
    lib = load()
    st = lib.hip_get_last_status()
    if st != 0:
        raise HipError(f"maidenx_hip status {st}: {lib.hip_status_string().decode()}")


def synchronize():
    rc = load().hip_synchronize()
    if rc != 0:
        raise HipError(f"hip_synchronize failed with {rc}")
    check()


NP_DTYPE = {"f32": np.float32, "bf16": np.uint16, "f16": np.uint16, "bool": np.uint8, "f64": np.float64, "i32": np.int32, "i64": np.int64}


class DeviceBuffer:
    """A device allocation of the backend (the analogue of the reference's CudaBuffer,
    crates/maidenx_core/src/buffer/cuda.rs:10-66): hip_malloc on creation, hip_free on drop."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        p = C.c_void_p()
        rc = load().hip_malloc(C.byref(p), max(self.nbytes, 1))
        if rc != 0:
            raise HipError("out of device memory" if rc == 2 else f"hip_malloc failed with {rc}")
        self.ptr = p.value

    @classmethod
    def from_numpy(cls, arr):
        arr = np.ascontiguousarray(arr)
        buf = cls(arr.nbytes)
        if arr.nbytes:
            rc = load().hip_memcpy_h2d(buf.ptr, arr.ctypes.data, arr.nbytes)
            if rc != 0:
                raise HipError(f"hip_memcpy_h2d failed with {rc}")
        return buf

    def to_numpy(self, dtype, count=None):
        dtype = np.dtype(dtype)
        n = self.nbytes // dtype.itemsize if count is None else int(count)
        out = np.empty(n, dtype=dtype)
        if out.nbytes:
            rc = load().hip_memcpy_d2h(out.ctypes.data, self.ptr, out.nbytes)
            if rc != 0:
                raise HipError(f"hip_memcpy_d2h failed with {rc}")
        return out

    def __del__(self):
        try:
            if getattr(self, "ptr", None) and _lib is not None:
                _lib.hip_free(self.ptr)
        except Exception:
            pass
        self.ptr = None


def _arg(a):
    if isinstance(a, DeviceBuffer):
        return a.ptr
    if isinstance(a, np.ndarray):     # host metadata
        return a.ctypes.data
    return a


def call(name, *args):
    """Call hip_<name> with DeviceBuffer / numpy-metadata / scalar arguments."""
    fn = getattr(load(), "hip_" + name)
    fn(*[_arg(a) for a in args])
