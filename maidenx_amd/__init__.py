"""maidenx_amd — MI355X (gfx950) compute backend for MaidenX.

The product is the C-ABI library `libmaidenx_hip.so` (HIP kernels, declared in
include/maidenx_hip.h) plus the host layer above it.  This package holds the sources
(`csrc/`), the build script (`build.py`) and a thin ctypes binding (`lib.py`).
"""
from . import lib  # noqa: F401
