"""ctypes binding of libprism_amd.so (the C ABI declared in include/prism_amd.h).

There is no fallback: if the library cannot be built or loaded, importing
callers get an exception, never a CPU path.
"""
from __future__ import annotations

import ctypes as C
import threading

from .build import LIB_PATH, ensure_built, ensure_vendor_built

# name -> (restype, argtypes); must list every function include/prism_amd.h declares.
SIGNATURES = {
    "prism_version": (C.c_char_p, []),
    "prism_last_error_string": (C.c_char_p, []),
    "prism_device_info": (C.c_int, [C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_int),
                                    C.POINTER(C.c_size_t), C.POINTER(C.c_size_t), C.c_char_p, C.c_size_t]),
    "prism_tile_coords": (C.c_int, [C.c_int, C.c_int, C.c_int, C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "prism_wave_regroup_i32": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_void_p]),
    "prism_add_m": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int32, C.c_size_t, C.c_void_p]),
    "prism_scan_workspace_bytes": (C.c_size_t, [C.c_size_t]),
    "prism_scan_workspace_init": (C.c_int, [C.c_void_p, C.c_size_t, C.c_void_p]),
    "prism_scan_status": (C.c_int, [C.c_void_p, C.c_size_t, C.c_void_p]),
    "prism_scan_i32": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_void_p]),
    "prism_scan_i32_static": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
    "prism_scan_i32_ex": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_uint,
                                    C.c_longlong, C.c_void_p]),
    "prism_scan_exclusive_i32": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_void_p]),
    "prism_scan_max_i32": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_void_p]),
    "prism_scan_min_i32": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_void_p]),
    "prism_segmented_scan_i32": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t,
                                           C.c_void_p]),
    "prism_segmented_scan_i32_ex": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t,
                                              C.c_uint, C.c_longlong, C.c_void_p]),
    "prism_scan_i64": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_void_p]),
    "prism_scan_i64_ex": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_uint, C.c_longlong,
                                    C.c_void_p]),
    "prism_launch_scan": (C.c_void_p, [C.c_size_t, C.c_void_p, C.c_void_p]),
    "prism_sgemm": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, C.c_void_p, C.c_void_p,
                              C.c_float, C.c_void_p, C.c_void_p]),
    "prism_sgemm_workspace_bytes": (C.c_size_t, [C.c_int, C.c_int, C.c_int]),
    "prism_sgemm_ws": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, C.c_void_p, C.c_void_p,
                                 C.c_float, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p]),
    "prism_sgemm_ws_plan": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_size_t, C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "prism_run_my_kernel": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_int, C.c_float, C.c_void_p,
                                      C.c_void_p, C.c_float, C.c_void_p]),
    "prism_gemm_bf16": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "prism_runmyh100": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
}

_lock = threading.Lock()
_lib = None


def load() -> C.CDLL:
    """Load (building first if the file is absent) and type every entry point."""
    global _lib
    with _lock:
        if _lib is None:
            path = ensure_built()
            lib = C.CDLL(str(path))
            for name, (restype, argtypes) in SIGNATURES.items():
                fn = getattr(lib, name)  # AttributeError if the build lacks a symbol
                fn.restype = restype
                fn.argtypes = argtypes
            _lib = lib
    return _lib


# The vendor-baseline library (prism_amd/csrc/vendor/vendor_baselines.hip): hipCUB, rocBLAS and hipBLASLt behind
# plain C entry points, for the evaluation sweeps and their tests. Not part of include/prism_amd.h.
VENDOR_SIGNATURES = {
    "vendor_scan_temp_bytes": (C.c_int, [C.c_size_t, C.POINTER(C.c_size_t)]),
    "vendor_scan_inclusive_sum": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_void_p]),
    "vendor_sgemm": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_float, C.c_void_p, C.c_void_p, C.c_float, C.c_void_p, C.c_void_p]),
    "vendor_gemm_bf16_f32": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
    "vendor_gemm_bf16_colmajor": (C.c_int, [C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]),
}
_vendor = None


def load_vendor() -> C.CDLL:
    """Load (building first if the file is absent) the vendor-baseline library."""
    global _vendor
    with _lock:
        if _vendor is None:
            lib = C.CDLL(str(ensure_vendor_built()))
            for name, (restype, argtypes) in VENDOR_SIGNATURES.items():
                fn = getattr(lib, name)
                fn.restype = restype
                fn.argtypes = argtypes
            _vendor = lib
    return _vendor


def last_error() -> str:
    return load().prism_last_error_string().decode("utf-8", "replace")


__all__ = ["load", "load_vendor", "last_error", "SIGNATURES", "VENDOR_SIGNATURES", "LIB_PATH"]
