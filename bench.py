#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME] [--no-configs]

Headline (BASELINE.json `metric`): fp32 SGEMM TFLOP/s at 8192^3 (alpha 1, beta 0.5,
kernel 5 = wave tile on fp32 MFMA); the same JSON line carries the int32 scan at 2^30,
the bf16 MFMA GEMM at 8192^3 and add_m at 2^24 under "also", each with its own roofline
object. A "step" is one launch of the workload's entry point through the C ABI with
inputs already resident in HBM. Timing: W untimed steps, then exactly K steps between
two HIP events on the launch stream, device-synchronised on both sides.

"also" further holds every other BASELINE configuration ("configs": kernels 1..6 at 1024..8192, the
tail shapes, the scan and bf16 sizes), timed with fewer steps, and add_m at 2^28 (2^24 fits the
memory-side cache).

Every timed workload first passes a parity gate on the same data: the GEMMs against an fp64 product
of the whole matrix formed on the device, the scan through its difference invariant over the whole
array, add_m element for element; a workload that fails the gate raises and reports nothing. Every
timed call's return code is checked.

cpu_baseline: numpy/OpenBLAS sgemm on all host cores at the headline size; the scalar CPU oracle
(oracle/prism_oracle.c, 1 core) on a bounded sample and numpy.cumsum are listed beside it.
Baselines, not targets.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

PEAK = {  # MI355X published peaks
    "hbm_GBps": 8000.0,
    "fp32_mfma_TFLOPs": 157.3,
    "bf16_mfma_TFLOPs": 2500.0,
}


ROOT = Path(__file__).resolve().parent
# Helpers shared with the tests live in tests/: the parity gate (fp64_referee), the tables under profiles/
# (profile_tables) and the streaming calibration kernels (calibrate_stream).
sys.path.insert(0, str(ROOT / "tests"))
from profile_tables import (measured_traffic, write_counter_table, write_eval_tables, write_kernel_trace_table,  # noqa: E402
                            write_traffic_table)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def _capi():
    """The C-ABI library and the current stream handle: timed loops call the entry points
    directly so that Python-side argument checks are not part of a step."""
    import torch
    from prism_amd import _lib
    return _lib.load(), torch.cuda.current_stream().cuda_stream


SETTLE_MS = 150.0  # untimed run of the workload before the warm-up steps, see time_steps


def time_steps(fn, steps: int, warmup: int):
    """Returns mean milliseconds per step, measured with HIP events on the current stream. `fn` is one
    call of a C-ABI entry point and returns its code (0 = ok); any other code raises after the loop.

    Before the W warm-up steps the workload runs untimed for SETTLE_MS: the chip's clock and power
    management take tens of milliseconds to settle under a new load (the first launches of the bf16
    GEMM after an idle or memory-bound phase measured up to 15 % off the sustained rate), and three
    sub-millisecond warm-up steps do not cover that."""
    import torch
    bad = 0
    t0 = time.perf_counter()
    while (time.perf_counter() - t0) * 1e3 < SETTLE_MS:
        bad |= fn() or 0
        torch.cuda.synchronize()
    for _ in range(warmup):
        bad |= fn() or 0
    torch.cuda.synchronize()
    beg = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    beg.record()
    for _ in range(steps):
        bad |= fn() or 0
    end.record()
    torch.cuda.synchronize()
    if bad:
        from prism_amd import _lib
        raise RuntimeError(f"a timed call returned an error code ({bad}): {_lib.last_error()}")
    return beg.elapsed_time(end) / steps


# -------------------------------------------------- full-matrix parity checks --
# The parity gate is the tests' own full-size check (tests/fp64_referee.py): every element against an fp64
# product formed on the device, which the GPU tests pin to the CPU oracle on sampled rows.
from fp64_referee import gemm_bf16_max_err_fp64, sgemm_max_err_fp64  # noqa: E402


# ------------------------------------------------------------------ sgemm --

def bench_sgemm(prism, M, N, K, alpha, beta, variant, steps, warmup, gate=True, with_workspace=False):
    """with_workspace: through prism_sgemm_ws with the workspace prism_sgemm_workspace_bytes asks for (kernel 5
    then cuts K across workgroups on skinny shapes); otherwise the reference-shaped prism_sgemm."""
    import torch
    g = torch.Generator(device="cuda")
    g.manual_seed(0)
    A = torch.rand((M, K), dtype=torch.float32, device="cuda", generator=g) * 2 - 1
    B = torch.rand((K, N), dtype=torch.float32, device="cuda", generator=g) * 2 - 1
    C0 = torch.rand((M, N), dtype=torch.float32, device="cuda", generator=g) * 2 - 1
    C = C0.clone()
    ws = torch.empty(max(prism.sgemm_workspace_size(M, N, K), 16), dtype=torch.uint8, device="cuda") if with_workspace else None
    if gate:
        prism.sgemm(M, N, K, alpha, A, B, beta, C, variant=variant, workspace=ws)
        err = sgemm_max_err_fp64(alpha, A, B, beta, C0, C)
        bound = 1e-5 * np.sqrt(K) + abs(beta) * 2**-22
        if not err <= bound:
            raise RuntimeError(f"sgemm kernel {variant} {M}x{N}x{K} failed the parity gate: err {err} > {bound}")
        C.copy_(C0)
    # Like the reference's sweep, C accumulates across repeats (evals/4090_sgemm/main.cu:199-203);
    # with |beta| < 1 it stays bounded.
    lib, st = _capi()
    a, b, c = A.data_ptr(), B.data_ptr(), C.data_ptr()
    if ws is None:
        ms = time_steps(lambda: lib.prism_sgemm(variant, M, N, K, alpha, a, b, beta, c, st), steps, warmup)
    else:
        w, wn = ws.data_ptr(), ws.numel()
        ms = time_steps(lambda: lib.prism_sgemm_ws(variant, M, N, K, alpha, a, b, beta, c, w, wn, st), steps, warmup)
    flops = 2.0 * M * N * K
    tflops = flops / (ms * 1e-3) / 1e12
    return {"ms": ms, "tflops": tflops,
            "roofline": {"bound": "mfma", "achieved": tflops, "peak": PEAK["fp32_mfma_TFLOPs"], "unit": "TFLOP/s",
                         "frac": tflops / PEAK["fp32_mfma_TFLOPs"],
                         "traffic": measured_traffic("sgemm", M) if M == N == K and variant == 5 else None}}


# ------------------------------------------------------------------- scan --

def bench_scan(prism, n, steps, warmup, gate=True, ticket_order=False):
    """ticket_order: tiles numbered by the reference's ticket counter (PRISM_SCAN_TICKET_ORDER) instead of by
    workgroup id, through prism_scan_i32_ex."""
    import torch
    g = torch.Generator(device="cuda")
    g.manual_seed(0)
    x = torch.randint(-1000, 1001, (n,), dtype=torch.int32, device="cuda", generator=g)
    out = torch.empty_like(x)
    ws = prism.new_scan_workspace(n)
    if gate:
        prism.scan(x, out, ws)
        torch.cuda.synchronize()
        ok = int(out[0]) == int(x[0])
        chunk = 1 << 26
        total = 0
        for s in range(0, n, chunk):
            e = min(n, s + chunk)
            lo = max(s, 1)
            ok = ok and bool(torch.equal(out[lo:e] - out[lo - 1:e - 1], x[lo:e]))
            total += int(x[s:e].sum(dtype=torch.int64))
        ok = ok and int(out[-1]) == ((total + 2**31) % 2**32) - 2**31
        if not ok:
            raise RuntimeError(f"scan n={n} failed the parity gate")
    # Out of place, so no restore is needed between steps. A step is the whole call: the kernel itself leaves
    # the workspace ready for the next call (the reference times two memsets per launch for that,
    # evals/4090_scan/main.cu:81-82).
    lib, st = _capi()
    xp, op, wp, wb = x.data_ptr(), out.data_ptr(), ws.data_ptr(), ws.numel()
    if ticket_order:
        ms = time_steps(lambda: lib.prism_scan_i32_ex(xp, op, n, wp, wb, 2, -1, st), steps, warmup)
    else:
        ms = time_steps(lambda: lib.prism_scan_i32(xp, op, n, wp, wb, st), steps, warmup)
    prism.scan_status(ws)  # raises if any timed call reported anything
    nbytes = 2.0 * 4 * n  # scan_harness.cuh:161
    gbps = nbytes / (ms * 1e-3) / 1e9
    return {"ms": ms, "GBps": gbps,
            "roofline": {"bound": "hbm", "achieved": gbps, "peak": PEAK["hbm_GBps"], "unit": "GB/s",
                         "frac": gbps / PEAK["hbm_GBps"], "traffic": measured_traffic("scan", n)}}


# ------------------------------------------------------------------ add_m --

def bench_add_m(prism, n, steps, warmup, gate=True):
    import torch
    g = torch.Generator(device="cuda")
    g.manual_seed(0)
    x = torch.randint(-2**20, 2**20, (n,), dtype=torch.int32, device="cuda", generator=g)
    y = torch.empty_like(x)
    if gate:
        prism.add_m(x, y, 7)
        torch.cuda.synchronize()
        if not torch.equal(y, x + 7):
            raise RuntimeError("add_m failed the parity gate")
    lib, st = _capi()
    xp, yp = x.data_ptr(), y.data_ptr()
    ms = time_steps(lambda: lib.prism_add_m(xp, yp, 7, n, st), steps, warmup)
    gbps = 8.0 * n / (ms * 1e-3) / 1e9
    return {"ms": ms, "GBps": gbps,
            "roofline": {"bound": "hbm", "achieved": gbps, "peak": PEAK["hbm_GBps"], "unit": "GB/s",
                         "frac": gbps / PEAK["hbm_GBps"], "traffic": measured_traffic("add_m", n)}}


# ------------------------------------------------------------ calibration --

CALIBRATION_KINDS = {0: "copy_packet_per_lane", 1: "copy_scan_tile_shape", 2: "read_only", 3: "write_only"}


def bench_calibration(steps, warmup):
    """What the memory system gives kernels that only move bytes (tests/native/calibrate_stream.hip): a 1 GiB copy in
    add_m's shape (the counter calibration) and, at the scan's size of 4 GiB per buffer, the copy in add_m's
    shape, the copy in the scan's tile shape, a read-only and a write-only stream."""
    import torch
    import calibrate_stream
    lib, st = calibrate_stream.load(), torch.cuda.current_stream().cuda_stream
    n = 1 << 30
    x = torch.randint(-1000, 1001, (n,), dtype=torch.int32, device="cuda")
    y = torch.empty_like(x)
    out = {}
    one_gib = 1 << 30
    ms = time_steps(lambda: lib.calibrate_stream(0, x.data_ptr(), y.data_ptr(), one_gib, st), steps, warmup)
    if not torch.equal(x[: one_gib // 4], y[: one_gib // 4]):
        raise RuntimeError("calibration copy is wrong")
    out["copy_1GiB"] = {"kernel": "calibrate_copy_packet_kernel", "bytes_read": one_gib, "bytes_written": one_gib,
                        "ms": ms, "GBps": 2.0 * one_gib / ms / 1e6}
    for kind, name in CALIBRATION_KINDS.items():
        ms = time_steps(lambda: lib.calibrate_stream(kind, x.data_ptr(), y.data_ptr(), 4 * n, st), steps, warmup)
        moved = (2 if kind < 2 else 1) * 4.0 * n
        out[name] = {"ms": ms, "GBps": moved / ms / 1e6, "frac_of_peak": moved / ms / 1e6 / PEAK["hbm_GBps"]}
    return out


# -------------------------------------------------------------- bf16 gemm --

def bench_gemm_bf16(prism, n, steps, warmup, gate=True):
    import torch
    g = torch.Generator(device="cuda")
    g.manual_seed(0)
    A = torch.randn((n, n), dtype=torch.float32, device="cuda", generator=g).to(torch.bfloat16)
    B = torch.randn((n, n), dtype=torch.float32, device="cuda", generator=g).to(torch.bfloat16)
    D = torch.empty((n, n), dtype=torch.float32, device="cuda")
    if gate:
        prism.gemm_bf16(A, B, D)
        err, ref_max = gemm_bf16_max_err_fp64(A, B, D)
        if not err <= 1e-3 * ref_max:
            raise RuntimeError(f"gemm_bf16 n={n} failed the parity gate: err {err}")
    lib, st = _capi()
    a, b, d = A.data_ptr(), B.data_ptr(), D.data_ptr()
    ms = time_steps(lambda: lib.prism_gemm_bf16(n, n, n, a, b, d, st), steps, warmup)
    tflops = 2.0 * n * n * n / (ms * 1e-3) / 1e12
    return {"ms": ms, "tflops": tflops,
            "roofline": {"bound": "mfma", "achieved": tflops, "peak": PEAK["bf16_mfma_TFLOPs"], "unit": "TFLOP/s",
                         "frac": tflops / PEAK["bf16_mfma_TFLOPs"], "traffic": measured_traffic("gemm_bf16", n)}}


def bench_runmyh100(prism, n, steps, warmup):
    """The same product through the reference harness's entry (evals/h100_bench/utils.cuh:504-533): bf16 column-major
    C[n * M + m], gated against the fp64 product at bf16's rounding step."""
    import torch
    g = torch.Generator(device="cuda")
    g.manual_seed(0)
    A = torch.randn((n, n), dtype=torch.float32, device="cuda", generator=g).to(torch.bfloat16)
    B = torch.randn((n, n), dtype=torch.float32, device="cuda", generator=g).to(torch.bfloat16)
    Cc = torch.empty((n, n), dtype=torch.bfloat16, device="cuda")
    lib, st = _capi()
    a, b, c = A.data_ptr(), B.data_ptr(), Cc.data_ptr()
    if lib.prism_runmyh100(n, n, n, a, b, c, None) != 0:
        raise RuntimeError("prism_runmyh100 failed")
    torch.cuda.synchronize()
    err, ref_max = gemm_bf16_max_err_fp64(A, B, Cc.T)   # C is column-major: its transpose view is M x N
    if not err <= 2.0 ** -8 * ref_max:
        raise RuntimeError(f"runmyh100 n={n} failed the parity gate: err {err}")
    ms = time_steps(lambda: lib.prism_runmyh100(n, n, n, a, b, c, None), steps, warmup)
    tflops = 2.0 * n * n * n / (ms * 1e-3) / 1e12
    return {"ms": ms, "tflops": tflops, "entry": "prism_runmyh100", "output": "bf16, column-major (the reference's)",
            "roofline": {"bound": "mfma", "achieved": tflops, "peak": PEAK["bf16_mfma_TFLOPs"], "unit": "TFLOP/s",
                         "frac": tflops / PEAK["bf16_mfma_TFLOPs"], "traffic": None}}


# ------------------------------------------------------- vendor libraries --

def bench_vendor(steps, warmup):
    """The ROCm libraries called directly (prism_amd/csrc/vendor/vendor_baselines.hip) on the headline problems,
    timed like the workloads above, in the same run: rocblas_sgemm at 8192^3 (alpha 1, beta 0.5),
    hipcub::DeviceScan::InclusiveSum at 2^30, hipBLASLt's bf16 matmul at 8192^3 with the fp32 row-major result of
    prism_gemm_bf16 and with the bf16 column-major result of the reference's harness (prism_runmyh100's).
    Comparison lines, like the cuBLAS / CUB lines of the reference's harnesses."""
    import ctypes

    import torch
    from prism_amd import _lib
    v, lib = _lib.load_vendor(), _lib.load()
    st = torch.cuda.current_stream().cuda_stream
    out = {}

    def checked(fn):
        def call():
            rc = fn()
            return 0 if rc == 0 else 1
        return call
    n = 8192
    g = torch.Generator(device="cuda")
    g.manual_seed(0)
    A = torch.rand((n, n), device="cuda", generator=g) * 2 - 1
    B = torch.rand((n, n), device="cuda", generator=g) * 2 - 1
    C = torch.rand((n, n), device="cuda", generator=g) * 2 - 1
    ms = time_steps(checked(lambda: v.vendor_sgemm(n, n, n, 1.0, A.data_ptr(), B.data_ptr(), 0.5, C.data_ptr(), st)), steps, warmup)
    out["rocblas_sgemm_8192"] = {"ms": ms, "tflops": 2.0 * n ** 3 / ms / 1e9}
    del A, B, C
    P = torch.randn((n, n), device="cuda", generator=g).to(torch.bfloat16)
    Q = torch.randn((n, n), device="cuda", generator=g).to(torch.bfloat16)
    D = torch.empty((n, n), dtype=torch.float32, device="cuda")
    Cc = torch.empty((n, n), dtype=torch.bfloat16, device="cuda")
    ms = time_steps(checked(lambda: v.vendor_gemm_bf16_f32(n, n, n, P.data_ptr(), Q.data_ptr(), D.data_ptr(), st)), steps, warmup)
    out["hipblaslt_bf16_8192_f32_out"] = {"ms": ms, "tflops": 2.0 * n ** 3 / ms / 1e9}
    ms = time_steps(checked(lambda: v.vendor_gemm_bf16_colmajor(n, n, n, P.data_ptr(), Q.data_ptr(), Cc.data_ptr(), st)), steps, warmup)
    out["hipblaslt_bf16_8192_bf16_colmajor_out"] = {"ms": ms, "tflops": 2.0 * n ** 3 / ms / 1e9}
    ms = time_steps(lambda: lib.prism_runmyh100(n, n, n, P.data_ptr(), Q.data_ptr(), Cc.data_ptr(), None), steps, warmup)
    out["ours_bf16_8192_bf16_colmajor_out"] = {"ms": ms, "tflops": 2.0 * n ** 3 / ms / 1e9, "entry": "prism_runmyh100"}
    del P, Q, D, Cc
    m = 1 << 30
    x = torch.randint(-1000, 1001, (m,), dtype=torch.int32, device="cuda")
    y = torch.empty_like(x)
    need = ctypes.c_size_t(0)
    if v.vendor_scan_temp_bytes(m, ctypes.byref(need)) != 0:
        raise RuntimeError("vendor_scan_temp_bytes failed")
    temp = torch.empty(max(need.value, 16), dtype=torch.uint8, device="cuda")
    ms = time_steps(checked(lambda: v.vendor_scan_inclusive_sum(x.data_ptr(), y.data_ptr(), m, temp.data_ptr(), temp.numel(), st)), steps, warmup)
    out["hipcub_inclusive_sum_2p30"] = {"ms": ms, "GBps": 8.0 * m / ms / 1e6}
    return out


def vendor_sgemm_tflops(M, N, K, alpha, beta, steps, warmup):
    """rocblas_sgemm called directly on one shape (seeded operands like bench_sgemm's), timed like a workload."""
    import torch
    from prism_amd import _lib
    v = _lib.load_vendor()
    st = torch.cuda.current_stream().cuda_stream
    g = torch.Generator(device="cuda")
    g.manual_seed(0)
    A = torch.rand((M, K), device="cuda", generator=g) * 2 - 1
    B = torch.rand((K, N), device="cuda", generator=g) * 2 - 1
    C = torch.rand((M, N), device="cuda", generator=g) * 2 - 1
    ms = time_steps(lambda: 0 if v.vendor_sgemm(M, N, K, alpha, A.data_ptr(), B.data_ptr(), beta, C.data_ptr(), st) == 0 else 1,
                    steps, warmup)
    return 2.0 * M * N * K / ms / 1e9


# ----------------------------------------------------------- CPU baselines --

def cpu_baseline_sgemm(n=8192, rows=4):
    """Oracle (scalar fmaf port, 1 core) on the first `rows` rows of the n^3 problem (about 2 s)."""
    import oracle
    A, B, Cm = oracle.gen_sgemm(rows, n, n, seed=0)
    t0 = time.perf_counter()
    oracle.sgemm_fma(1.0, A, B, 0.5, Cm)
    dt = time.perf_counter() - t0
    return {"value": 2.0 * rows * n * n / dt / 1e12, "unit": "TFLOP/s", "cores": 1, "kind": "port",
            "sample": f"oracle_sgemm_fma on the first {rows} rows of C ({rows}x{n}x{n}), {dt:.1f} s"}


def cpu_blas_sgemm(n=8192):
    """numpy/OpenBLAS sgemm on all host cores at the headline size (one untimed product first)."""
    rng = np.random.default_rng(0)
    A = rng.random((n, n), dtype=np.float32)
    B = rng.random((n, n), dtype=np.float32)
    Cm = rng.random((n, n), dtype=np.float32)
    A[:1024] @ B  # warm: thread pool and pages
    t0 = time.perf_counter()
    np.float32(1.0) * (A @ B) + np.float32(0.5) * Cm
    dt = time.perf_counter() - t0
    threads = None
    try:
        from threadpoolctl import threadpool_info
        threads = max((p.get("num_threads", 0) for p in threadpool_info()), default=None)
    except Exception:
        pass
    return {"value": 2.0 * n**3 / dt / 1e12, "unit": "TFLOP/s", "cores": threads or os.cpu_count(),
            "kind": "port", "library": "numpy/OpenBLAS sgemm (the reference holds no CPU GEMM)",
            "sample": f"the whole {n}^3 problem once, alpha*(A@B)+beta*C, {dt:.2f} s", "os_cpu_count": os.cpu_count()}


def cpu_baseline_scan(n=1 << 28):
    import oracle
    x = oracle.gen_scan(n, seed=0)
    t0 = time.perf_counter()
    oracle.scan_cpu(x)
    dt = time.perf_counter() - t0
    t1 = time.perf_counter()
    np.cumsum(x, dtype=np.int32)
    dt_np = time.perf_counter() - t1
    return {"value": 8.0 * n / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"oracle_scan_cpu (serial loop of scan_harness.cuh:30-36) on n=2^{n.bit_length() - 1}, {dt:.2f} s",
            "numpy_cumsum_GBps": 8.0 * n / dt_np / 1e9}


def cpu_baseline_add_m(n=1 << 24):
    import oracle
    x = oracle.gen_add_m(n, seed=0)
    t0 = time.perf_counter()
    oracle.add_m(x, 7)
    dt = time.perf_counter() - t0
    t1 = time.perf_counter()
    x + np.int32(7)
    dt_np = time.perf_counter() - t1
    return {"value": 8.0 * n / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"oracle_add_m on n=2^24, {dt * 1e3:.1f} ms", "numpy_GBps": 8.0 * n / dt_np / 1e9}


# ------------------------------------------------------------------- main --

def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--workload", default="all", choices=["all", "sgemm", "scan", "gemm_bf16", "add_m", "calibrate"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-vendor", action="store_true", help="skip the vendor-library comparison lines (also.vendor_libraries)")
    ap.add_argument("--no-configs", action="store_true",
                    help="skip the table of the other BASELINE configurations (also.configs)")
    ap.add_argument("--traffic-summary", metavar="DIR", default=None,
                    help="no GPU work: summarise the rocprofv3 --pmc outputs in DIR into profiles/hbm_traffic.md")
    ap.add_argument("--trace-summary", metavar="DIR", default=None,
                    help="no GPU work: summarise the rocprofv3 --kernel-trace --stats output in DIR into "
                         "profiles/bench_all_kernels_kernel_trace.md")
    ap.add_argument("--counter-summary", metavar="DIR", default=None,
                    help="no GPU work: summarise three rocprofv3 --pmc runs (p1, p2, p3) in DIR into profiles/kernel_counters.md")
    ap.add_argument("--eval-summary", metavar="DIR", default=None,
                    help="no GPU work: summarise eval_report.txt / eval_generated.txt in DIR (outputs of "
                         "`python -m prism_amd.eval_report [generated]`) into profiles/eval_sweeps.md")
    args = ap.parse_args()
    if args.eval_summary:
        return write_eval_tables(args.eval_summary)
    if args.counter_summary:
        return write_counter_table(args.counter_summary)
    if args.traffic_summary:
        return write_traffic_table(args.traffic_summary)
    if args.trace_summary:
        return write_kernel_trace_table(args.trace_summary)
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (the path has no multi-GPU part); run with --gpus 1",
              file=sys.stderr)
        return 2

    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 1
    import prism_amd as prism
    info = prism.device_info()
    log(f"device: {info}")
    K, W = args.steps, args.warmup
    want = lambda w: args.workload in ("all", w)

    if args.workload == "calibrate":
        # Plain streaming kernels of known size (tests/native/calibrate_stream.hip): the copy of 1 GiB (kind 0) is what the
        # FETCH_SIZE / WRITE_SIZE counters of a `rocprofv3 --pmc` run of this script are scaled by; all four kinds
        # at 4 GiB are the ceiling the streaming workloads are compared with.
        print(json.dumps({"workload": "calibrate", **bench_calibration(K, W)}), flush=True)
        return 0

    res = {}
    if want("sgemm"):
        res["sgemm"] = bench_sgemm(prism, 8192, 8192, 8192, 1.0, 0.5, 5, K, W)
        log("sgemm 8192^3 kernel 5:", res["sgemm"])
    if want("scan"):
        res["scan"] = bench_scan(prism, 1 << 30, K, W)
        log("scan 2^30:", res["scan"])
        res["scan_ticket_order"] = bench_scan(prism, 1 << 30, K, W, gate=False, ticket_order=True)
        res["scan_ticket_order"]["note"] = ("the same scan with tiles numbered by the reference's ticket counter "
                                            "(examples/scan.py:88-99) instead of by workgroup id")
        log("scan 2^30, ticket order:", res["scan_ticket_order"])
    if want("gemm_bf16"):
        res["gemm_bf16"] = bench_gemm_bf16(prism, 8192, K, W)
        log("gemm_bf16 8192^3:", res["gemm_bf16"])
        res["gemm_bf16_runmyh100"] = bench_runmyh100(prism, 8192, K, W)
        log("gemm_bf16 8192^3 through prism_runmyh100:", res["gemm_bf16_runmyh100"])
    if want("add_m"):
        res["add_m"] = bench_add_m(prism, 1 << 24, max(K, 50), W)
        log("add_m 2^24:", res["add_m"])

    if args.workload == "all" or args.workload in ("scan", "add_m"):
        res["hbm_calibration"] = bench_calibration(K, W)
        log("streaming calibration:", res["hbm_calibration"])
    if want("add_m"):
        res["add_m_2p28"] = bench_add_m(prism, 1 << 28, K, W)
        res["add_m_2p28"]["note"] = "x and y are 2 GiB together: beyond the 256 MiB memory-side cache"
        res["add_m"]["note"] = "x and y are 128 MiB together and fit the 256 MiB memory-side cache: not an HBM-bound figure"
        log("add_m 2^28:", res["add_m_2p28"])

    if args.workload == "all" and not args.no_vendor:
        res["vendor_libraries"] = bench_vendor(K, W)
        log("vendor libraries:", res["vendor_libraries"])

    # Every other BASELINE configuration, with fewer steps (kernel 1 at 8192^3 takes 0.35 s a step): a table
    # under "also.configs" of the JSON line, each entry parity-gated like the headline workloads.
    configs = {}
    if args.workload == "all" and not args.no_configs:
        for n in (1024, 2048, 4096, 8192):
            for v in (1, 2, 3, 6, 4, 5):
                if n == 8192 and v == 5:
                    continue  # the headline
                k, w = (2, 1) if (n >= 4096 and v in (1, 2, 3)) else (5, 1) if n >= 4096 else (10, 2)
                r = bench_sgemm(prism, n, n, n, 1.0, 0.5, v, k, w)
                configs[f"sgemm_k{v}_{n}"] = {"ms": r["ms"], "tflops": r["tflops"], "frac": r["roofline"]["frac"], "steps": k}
                log(f"  sgemm kernel {v} {n}^3: {r['ms']:.3f} ms  {r['tflops']:.2f} TFLOP/s  "
                    f"({100 * r['roofline']['frac']:.1f}% of fp32 MFMA peak)")
        for (M, N, Kd) in ((4096, 4096, 128), (128, 4096, 4096), (8191, 4097, 1023), (16384, 16384, 512)):
            r = bench_sgemm(prism, M, N, Kd, 1.0, 0.0, 5, 10, 2)
            configs[f"sgemm_k5_{M}x{N}x{Kd}"] = {"ms": r["ms"], "tflops": r["tflops"], "frac": r["roofline"]["frac"], "steps": 10}
            log(f"  sgemm kernel 5 {M}x{N}x{Kd}: {r['ms']:.3f} ms  {r['tflops']:.2f} TFLOP/s")
        # Shapes whose tiles do not fill whole rounds of the CUs, through the reference-shaped entry and through the
        # workspace form (prism_sgemm_ws: K ranges shared between all CUs); the plan query says that the shared
        # form is what the "with_workspace" rows measured.
        for (M, N, Kd) in ((128, 4096, 4096), (5120, 5120, 5120), (4352, 4352, 4352), (3200, 3200, 3200)):
            name = f"sgemm_k5_{M}x{N}x{Kd}"
            if name not in configs:
                r = bench_sgemm(prism, M, N, Kd, 1.0, 0.0, 5, 10, 2)
                configs[name] = {"ms": r["ms"], "tflops": r["tflops"], "frac": r["roofline"]["frac"], "steps": 10}
                log(f"  sgemm kernel 5 {M}x{N}x{Kd}: {r['ms']:.3f} ms  {r['tflops']:.2f} TFLOP/s")
            groups, shared = prism.sgemm_workspace_plan(M, N, Kd, prism.sgemm_workspace_size(M, N, Kd))
            if groups == 0:
                continue  # nothing would be shared for this shape (3200^3: fewer tiles than CUs)
            r = bench_sgemm(prism, M, N, Kd, 1.0, 0.0, 5, 10, 2, with_workspace=True)
            configs[name + "_with_workspace"] = {"ms": r["ms"], "tflops": r["tflops"], "frac": r["roofline"]["frac"], "steps": 10,
                                                 "entry": "prism_sgemm_ws", "workgroups_sharing": groups, "tiles_shared": shared}
            log(f"  sgemm kernel 5 {M}x{N}x{Kd} with workspace ({shared} tiles shared by {groups} workgroups): "
                f"{r['ms']:.3f} ms  {r['tflops']:.2f} TFLOP/s")
        if not args.no_vendor:   # rocblas_sgemm on the same shapes, same run and protocol
            for (M, N, Kd) in ((4096, 4096, 128), (128, 4096, 4096), (8191, 4097, 1023), (16384, 16384, 512),
                               (5120, 5120, 5120), (4352, 4352, 4352), (3200, 3200, 3200)):
                configs[f"sgemm_k5_{M}x{N}x{Kd}"]["rocblas_sgemm_tflops"] = vendor_sgemm_tflops(M, N, Kd, 1.0, 0.0, 10, 2)
                log(f"  rocblas_sgemm {M}x{N}x{Kd}: {configs[f'sgemm_k5_{M}x{N}x{Kd}']['rocblas_sgemm_tflops']:.2f} TFLOP/s")
        for p in (20, 24, 28):
            r = bench_scan(prism, 1 << p, 20, 3)
            configs[f"scan_2p{p}"] = {"ms": r["ms"], "GBps": r["GBps"], "frac": r["roofline"]["frac"], "steps": 20}
            log(f"  scan 2^{p}: {r['ms']:.4f} ms  {r['GBps']:.1f} GB/s ({100 * r['roofline']['frac']:.1f}% of HBM peak)")
        for n in (4096, 16384):
            r = bench_gemm_bf16(prism, n, 8, 2)
            configs[f"gemm_bf16_{n}"] = {"ms": r["ms"], "tflops": r["tflops"], "frac": r["roofline"]["frac"], "steps": 8}
            log(f"  gemm_bf16 {n}^3: {r['ms']:.3f} ms  {r['tflops']:.1f} TFLOP/s "
                f"({100 * r['roofline']['frac']:.1f}% of bf16 MFMA peak)")

    cpu = {}
    if not args.no_cpu_baseline:
        if want("sgemm"):
            cpu["sgemm"] = cpu_blas_sgemm()
            cpu["sgemm_scalar_oracle"] = cpu_baseline_sgemm()
        if want("scan"):
            cpu["scan"] = cpu_baseline_scan()
        if want("add_m"):
            cpu["add_m"] = cpu_baseline_add_m()
        log("cpu baselines:", cpu)

    head_name = "sgemm" if "sgemm" in res else next(iter(res))
    head = res[head_name]
    if head_name in ("sgemm", "gemm_bf16"):
        metric = {"sgemm": "SGEMM TFLOP/s @8192^3 fp32", "gemm_bf16": "bf16 GEMM TFLOP/s @8192^3"}[head_name]
        value, unit = head["tflops"], "TFLOP/s"
        dtype = "f32" if head_name == "sgemm" else "bf16"
    else:
        metric = {"scan": "int32 scan GB/s @2^30", "add_m": "add_m GB/s @2^24"}[head_name]
        value, unit = head["GBps"], "GB/s"
        dtype = "i32"
    workload = {"sgemm": "sgemm M=N=K=8192 alpha=1 beta=0.5 kernel 5 (wave tile, fp32 MFMA)",
                "scan": "inclusive scan int32 n=2^30, values in [-1000,1000]",
                "gemm_bf16": "D=A@B^T bf16 in, fp32 out, M=N=K=8192",
                "add_m": "y=x+7 int32 n=2^24"}[head_name]
    line = {
        "metric": metric, "value": value, "unit": unit, "n_gpus": 1, "steps": K, "warmup": W, "settle_ms": SETTLE_MS,
        "ms_per_step": head["ms"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": dtype, "data": "synthetic",
        "config": {"workload": workload, "device": info["name"], "cu_count": info["cu_count"]},
        "roofline": head["roofline"],
        "cpu_baseline": cpu.get(head_name),
        "also": {**{k: v for k, v in res.items() if k != head_name}, **({"configs": configs} if configs else {})},
        "cpu_baselines_also": {k: v for k, v in cpu.items() if k != head_name},
    }
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
