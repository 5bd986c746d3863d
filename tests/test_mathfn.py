"""CPU: the backend's exp / tanh / expm1 (maidenx_amd/csrc/mathfn.hpp, compiled for the host) return
the same bits as the platform libm that the reference's CPU path calls.  The default run walks
every 61st f32 bit pattern (70 M inputs per function); MATHFN_EXHAUSTIVE=1 walks all 2^32."""
import ctypes as C
import os
import subprocess

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "native", "mathfn_host.cpp")
LIB = os.path.join(HERE, "native", "libmathfn_host.so")


@pytest.fixture(scope="module")
def mathfn():
    hdr = os.path.join(HERE, "..", "maidenx_amd", "csrc", "mathfn.hpp")
    if not os.path.exists(LIB) or os.path.getmtime(LIB) < max(os.path.getmtime(SRC), os.path.getmtime(hdr)):
        subprocess.run(["g++", "-O2", "-shared", "-fPIC", "-fopenmp", "-ffp-contract=off", "-mfma", SRC, "-o", LIB, "-lm"], check=True)
    lib = C.CDLL(LIB)
    lib.mathfn_mismatches.argtypes = [C.c_int, C.c_uint32, C.c_uint32, C.c_long, C.POINTER(C.c_float)]
    lib.mathfn_mismatches.restype = C.c_long
    return lib


@pytest.mark.parametrize("which,name", [(0, "exp"), (1, "tanh"), (2, "expm1")])
def test_restatement_is_bit_identical_to_libm(mathfn, which, name):
    stride, count = (1, 1 << 32) if os.environ.get("MATHFN_EXHAUSTIVE") else (61, (1 << 32) // 61)
    bad_x = C.c_float(0)
    bad = mathfn.mathfn_mismatches(which, 0, stride, count, C.byref(bad_x))
    assert bad == 0, f"{name}: {bad} mismatching inputs, e.g. x={bad_x.value!r}"


def test_special_values(mathfn):
    mathfn.mathfn_eval.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_long]
    x = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 88.8, -104.0, -103.5, 1e-40, -1e-40], dtype=np.float32)
    y = np.empty_like(x)
    mathfn.mathfn_eval(0, x.ctypes.data, y.ctypes.data, x.size)
    with np.errstate(all="ignore"):
        assert np.array_equal(y, np.exp(x.astype(np.float64)).astype(np.float32), equal_nan=True)
    mathfn.mathfn_eval(1, x.ctypes.data, y.ctypes.data, x.size)
    assert np.array_equal(y.view(np.uint32)[:4], np.tanh(x[:4]).view(np.uint32))     # signed zeros and +-1 at infinity
