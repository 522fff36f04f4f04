"""Loader of the streaming calibration kernels (tests/native/calibrate_stream.hip -> libcalibrate_stream.so).

A measurement aid for bench.py and the GPU tests: plain copy / read / write kernels of known size, kept out of
libprism_amd.so and its header. `build()` compiles for gfx950 with the product library's flags (the driver's
build step calls it, so the library travels to the GPU box with the tree); `load()` compiles only when the
library is missing.
"""
from __future__ import annotations

import ctypes as C
import sys
from pathlib import Path

HERE = Path(__file__).resolve().parent
SOURCE = HERE / "native" / "calibrate_stream.hip"
LIB_PATH = HERE / "native" / "libcalibrate_stream.so"
_lib = None


def build() -> Path:
    root = str(HERE.parent)
    if root not in sys.path:
        sys.path.insert(0, root)
    from prism_amd import build as b
    b._run([b.hipcc_path(), *b.HIPCC_FLAGS, "-shared", "-o", str(LIB_PATH), str(SOURCE)], verbose=False)
    return LIB_PATH


def load() -> C.CDLL:
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            build()
        _lib = C.CDLL(str(LIB_PATH))
        _lib.calibrate_stream.restype = C.c_int
        _lib.calibrate_stream.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]
    return _lib
