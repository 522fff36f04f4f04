"""ctypes face of oracle/prism_oracle.c plus numpy restatements.

TEST INFRASTRUCTURE ONLY (see the header of prism_oracle.c). The C functions are
the oracle proper; the ``np_*`` functions are independent numpy formulations
used to pin the C code and as the "numpy" CPU baselines.
"""
from __future__ import annotations

import ctypes as C
import subprocess
from pathlib import Path

import numpy as np

ORACLE_DIR = Path(__file__).resolve().parent
LIB = ORACLE_DIR / "liboracle.so"

_lib = None


def build(force: bool = False) -> Path:
    """Compile liboracle.so with gcc through oracle/Makefile."""
    if force and LIB.exists():
        LIB.unlink()
    proc = subprocess.run(["make", "-C", str(ORACLE_DIR), "liboracle.so"], capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("building the oracle failed:\n" + proc.stdout + proc.stderr)
    return LIB


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not LIB.exists():
            build()
        L = C.CDLL(str(LIB))
        vp, sz, i32, f32 = C.c_void_p, C.c_size_t, C.c_int32, C.c_float
        L.oracle_add_m.argtypes = [vp, vp, i32, sz]
        L.oracle_add_m.restype = None
        L.oracle_scan_cpu.argtypes = [sz, vp, vp]
        L.oracle_scan_cpu.restype = None
        L.oracle_scan_exclusive_cpu.argtypes = [sz, vp, vp]
        L.oracle_scan_exclusive_cpu.restype = None
        L.oracle_segmented_scan_cpu.argtypes = [sz, vp, vp, vp]
        L.oracle_segmented_scan_cpu.restype = None
        L.oracle_scan_i64_cpu.argtypes = [sz, vp, vp]
        L.oracle_scan_i64_cpu.restype = None
        L.oracle_scan_max_cpu.argtypes = [sz, vp, vp]
        L.oracle_scan_max_cpu.restype = None
        L.oracle_scan_lookback.argtypes = [sz, vp, C.c_uint]
        L.oracle_scan_lookback.restype = sz
        L.oracle_sgemm_fma.argtypes = [C.c_int, C.c_int, C.c_int, f32, vp, vp, f32, vp]
        L.oracle_sgemm_fma.restype = None
        L.oracle_sgemm_f64.argtypes = [C.c_int, C.c_int, C.c_int, f32, vp, vp, f32, vp, vp]
        L.oracle_sgemm_f64.restype = None
        L.oracle_f32_to_bf16.argtypes = [f32]
        L.oracle_f32_to_bf16.restype = C.c_uint16
        L.oracle_bf16_to_f32.argtypes = [C.c_uint16]
        L.oracle_bf16_to_f32.restype = f32
        L.oracle_f32_to_bf16_array.argtypes = [vp, vp, sz]
        L.oracle_f32_to_bf16_array.restype = None
        L.oracle_gemm_bf16_f64.argtypes = [C.c_int, C.c_int, C.c_int, vp, vp, vp]
        L.oracle_gemm_bf16_f64.restype = None
        _lib = L
    return _lib


def _c(a: np.ndarray, dtype) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=dtype)
    return a


def _p(a: np.ndarray) -> int:
    return a.ctypes.data


# ------------------------------------------------------------------- add_m --

def add_m(x: np.ndarray, m: int) -> np.ndarray:
    x = _c(x, np.int32)
    y = np.empty_like(x)
    m = ((int(m) + 2**31) % 2**32) - 2**31
    lib().oracle_add_m(_p(x), _p(y), m, x.size)
    return y


def np_add_m(x: np.ndarray, m: int) -> np.ndarray:
    """Same sum through 64-bit unsigned arithmetic reduced modulo 2^32."""
    wide = x.view(np.uint32).astype(np.uint64) + np.uint64(int(m) % 2**32)
    return (wide % np.uint64(2**32)).astype(np.uint32).view(np.int32)


# -------------------------------------------------------------------- scan --

def scan_cpu(x: np.ndarray) -> np.ndarray:
    """Serial uint32 inclusive scan; int32 input gives the int32 view of the same bits."""
    dt = x.dtype
    xu = _c(x, dt).view(np.uint32)
    out = np.empty_like(xu)
    lib().oracle_scan_cpu(xu.size, _p(xu), _p(out))
    return out.view(dt)


def scan_exclusive_cpu(x: np.ndarray) -> np.ndarray:
    """Serial uint32 exclusive scan: out[0] = 0, out[i] = x[0] + ... + x[i-1]."""
    dt = x.dtype
    xu = _c(x, dt).view(np.uint32)
    out = np.empty_like(xu)
    lib().oracle_scan_exclusive_cpu(xu.size, _p(xu), _p(out))
    return out.view(dt)


def scan_max_cpu(x: np.ndarray) -> np.ndarray:
    """Serial running maximum of int32: out[i] = max(x[0], ..., x[i])."""
    xi = _c(x, np.int32)
    out = np.empty_like(xi)
    lib().oracle_scan_max_cpu(xi.size, _p(xi), _p(out))
    return out


def segmented_scan_cpu(x: np.ndarray, heads: np.ndarray) -> np.ndarray:
    """Serial uint32 inclusive scan that starts again at every element whose head flag is non-zero."""
    dt = x.dtype
    xu = _c(x, dt).view(np.uint32)
    h = _c(heads, np.uint8)
    assert h.size == xu.size
    out = np.empty_like(xu)
    lib().oracle_segmented_scan_cpu(xu.size, _p(xu), _p(h), _p(out))
    return out.view(dt)


def np_segmented_scan(x: np.ndarray, heads: np.ndarray) -> np.ndarray:
    """The same through one global cumulative sum: out[i] = S[i] - S[start(i) - 1] modulo 2^32, where start(i)
    is the last head at or before i."""
    xu = x.view(np.uint32).astype(np.uint64)
    S = np.cumsum(xu)  # exact in 64 bits for fewer than 2^32 elements
    idx = np.arange(x.size)
    h = np.asarray(heads) != 0
    if x.size:
        h = h.copy()
        h[0] = True
    start = np.maximum.accumulate(np.where(h, idx, 0))
    before = np.where(start > 0, S[np.maximum(start - 1, 0)], 0)
    return ((S - before) % np.uint64(2**32)).astype(np.uint32).view(x.dtype)


def scan_i64_cpu(x: np.ndarray) -> np.ndarray:
    """Serial inclusive scan of 64-bit elements modulo 2^64."""
    dt = x.dtype
    xu = _c(x, dt).view(np.uint64)
    out = np.empty_like(xu)
    lib().oracle_scan_i64_cpu(xu.size, _p(xu), _p(out))
    return out.view(dt)


def gen_heads(n: int, mean_segment: float, seed: int = 0) -> np.ndarray:
    """Head flags (uint8, values 0 / 1 / 255) with segments of the given mean length."""
    rng = np.random.default_rng(seed)
    h = (rng.random(n) < 1.0 / mean_segment).astype(np.uint8)
    h[rng.random(n) < 0.5] *= np.uint8(255)  # any non-zero byte is a head
    return h


def scan_lookback(x: np.ndarray, stall_every: int = 0) -> np.ndarray:
    """Block-structured restatement (16384-element blocks); a tail past the last block is left as is."""
    dt = x.dtype
    buf = np.array(x, dtype=dt, copy=True).view(np.uint32)
    lib().oracle_scan_lookback(buf.size, _p(buf), stall_every)
    return buf.view(dt)


def np_scan(x: np.ndarray) -> np.ndarray:
    return np.cumsum(x, dtype=x.dtype)


# ------------------------------------------------------------------- sgemm --

def sgemm_fma(alpha, A, B, beta, Cin) -> np.ndarray:
    A = _c(A, np.float32); B = _c(B, np.float32)
    M, K = A.shape; K2, N = B.shape
    assert K == K2
    Cout = np.array(Cin, dtype=np.float32, copy=True, order="C").reshape(M, N)
    lib().oracle_sgemm_fma(M, N, K, alpha, _p(A), _p(B), beta, _p(Cout))
    return Cout


def sgemm_f64(alpha, A, B, beta, Cin=None) -> np.ndarray:
    A = _c(A, np.float32); B = _c(B, np.float32)
    M, K = A.shape; K2, N = B.shape
    assert K == K2
    out = np.empty((M, N), dtype=np.float64)
    cin = None if Cin is None else _c(Cin, np.float32)
    assert beta == 0 or cin is not None
    lib().oracle_sgemm_f64(M, N, K, alpha, _p(A), _p(B), beta, 0 if cin is None else _p(cin), _p(out))
    return out


def np_sgemm_f64(alpha, A, B, beta, Cin=None) -> np.ndarray:
    ab = np.float64(np.float32(alpha)) * (A.astype(np.float64) @ B.astype(np.float64))
    if beta == 0:
        return ab
    return ab + np.float64(np.float32(beta)) * Cin.astype(np.float64)


def sgemm_tolerance(K: int, A: np.ndarray, B: np.ndarray) -> float:
    """Max abs error allowed against the fp64 product: 1e-5 * sqrt(K) * max|A| * max|B|."""
    return 1e-5 * np.sqrt(max(K, 1)) * float(np.abs(A).max(initial=0.0)) * float(np.abs(B).max(initial=0.0))


# --------------------------------------------------------------- bf16 gemm --

def f32_to_bf16(a: np.ndarray) -> np.ndarray:
    a = _c(a, np.float32)
    out = np.empty(a.shape, dtype=np.uint16)
    lib().oracle_f32_to_bf16_array(_p(a), _p(out), a.size)
    return out


def np_f32_to_bf16(a: np.ndarray) -> np.ndarray:
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    return r


def bf16_to_f32(h: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(h, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def gemm_bf16_f64(A16: np.ndarray, B16: np.ndarray) -> np.ndarray:
    A16 = _c(A16, np.uint16); B16 = _c(B16, np.uint16)
    M, K = A16.shape; N, K2 = B16.shape
    assert K == K2
    D = np.empty((M, N), dtype=np.float64)
    lib().oracle_gemm_bf16_f64(M, N, K, _p(A16), _p(B16), _p(D))
    return D


def np_gemm_bf16_f64(A16: np.ndarray, B16: np.ndarray) -> np.ndarray:
    return bf16_to_f32(A16).astype(np.float64) @ bf16_to_f32(B16).astype(np.float64).T


# ------------------------------------------------- seeded workload generators

def gen_add_m(n: int, seed: int = 0) -> np.ndarray:
    return np.random.default_rng(seed).integers(-2**20, 2**20, n, dtype=np.int32)


def gen_scan(n: int, seed: int = 0) -> np.ndarray:
    return np.random.default_rng(seed).integers(-1000, 1001, n, dtype=np.int32)


def gen_scan_reference_style(n: int, seed: int = 0xCA7CAFE) -> np.ndarray:
    """U{0..100} uint32, the distribution of the reference's own scan tests
    (evals/4090_scan/scan_harness.cuh:170-178); the generator differs (numpy PCG64, not mt19937)."""
    return np.random.default_rng(seed).integers(0, 101, n, dtype=np.uint32)


def gen_sgemm(M: int, N: int, K: int, seed: int = 0):
    rng = np.random.default_rng(seed)
    A = (rng.random((M, K), dtype=np.float32) * 2 - 1).astype(np.float32)
    B = (rng.random((K, N), dtype=np.float32) * 2 - 1).astype(np.float32)
    Cm = (rng.random((M, N), dtype=np.float32) * 2 - 1).astype(np.float32)
    return A, B, Cm


def gen_gemm_bf16(M: int, N: int, K: int, seed: int = 0):
    rng = np.random.default_rng(seed)
    A = np_f32_to_bf16(rng.standard_normal((M, K), dtype=np.float32))
    B = np_f32_to_bf16(rng.standard_normal((N, K), dtype=np.float32))
    return A, B
