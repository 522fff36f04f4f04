"""Evaluation sweeps in the reference harnesses' own methodology and text format.

    python -m prism_amd.eval_report [sgemm] [scan] [h100]      (default: all three)
    python -m prism_amd.eval_report generated                  (the same three sweeps over kernels generated from the DSL)

The counterpart of the reference's three benchmark mains, so that the text it
prints can be fed to the reference's plotting script unchanged:

  sgemm  evals/4090_sgemm/main.cu:43,154-217  sizes 256..8192, alpha 0.5, beta 3.0, 10 back-to-back
         launches between two events, GFLOPS = 2 m n k / t; blocks "[cuBLAS FP32]" / "[My Kernel k]"
         (parsed by evals/plot_results.py:37-79)
  scan   evals/4090_scan/bench.cu:157-262     n = 2^20..2^30, best wall-clock of launch + device sync over
         repeats until 500 ms have elapsed, GB/s = n * 4 * 2 / t; table "Size | CUB ... | Ours ..."
         (parsed by plot_results.py:82-108)
  h100   evals/h100_bench/main.cu:112-167     8 back-to-back launches between two events, TFLOPS;
         lines "Kernel: ..." / "cuBLAS: ..." (parsed by plot_results.py:18-34)

The vendor-library slots ("cuBLAS", "CUB") are filled by the ROCm libraries called directly, the way the
harnesses call theirs: rocblas_sgemm, a hipBLASLt bf16 matmul and hipcub::DeviceScan::InclusiveSum, behind the
C entry points of prism_amd/csrc/vendor/vendor_baselines.hip (a library of its own, built by prism_amd.build).
They are comparison lines, like the reference's.

`generated` runs the same protocols over the kernels that prism_amd.hipgen prints from the example programs
(prism_amd/examples), which is what the reference's figures show for its own back-end: "My Kernel" 1..5 are
naive_sgemm, remapped_sgemm, tiled_sgemm<32>, vector_tile_sgemm<128,128,8,8,8> and, on the fp32 matrix
instruction, pipelined_sgemm from 4096 up and handed_over_sgemm (the producer / consumer kernel) at 1024 and 2048
(smaller sizes, which neither takes, are left out), the scan is lookback_scan_striped, and "Kernel:" in the bf16
sweep is pipelined_gemm_bf16 from 4096 up and handed_over_gemm_big below (fp32 row-major output, where the
reference's kernel writes bf16 column-major). The kernels are compiled for gfx950 on the spot.
"""
from __future__ import annotations

import sys
import time

SGEMM_SIZES = (256, 512, 1024, 2048, 4096, 8192)            # evals/4090_sgemm/main.cu:43
SCAN_LOG2_SIZES = tuple(range(20, 31))                       # evals/4090_scan/bench.cu:157-169
H100_SIZES = (2048, 4096, 6144, 8192, 12288, 16384)          # evals/run_h100.sh:12


# ------------------------------------------------------------- formatting --

def sgemm_line(seconds_per_call: float, gflops: float, size: int) -> str:
    # printf format of evals/4090_sgemm/main.cu:182-186
    return ("Average elapsed time: (%7.6f) s, performance: (%7.1f) GFLOPS. size: (%ld)." % (seconds_per_call, gflops, size))


def h100_line(who: str, seconds_per_call: float, tflops: float, size: int) -> str:
    # printf format of evals/h100_bench/main.cu:149-152 ("Kernel:" / "cuBLAS:")
    return ("%s  Average elapsed time: (%7.6f) s, performance: (%7.1f) TFLOPS. size: (%ld)." % (who, seconds_per_call, tflops, size))


def scan_header() -> str:
    # evals/4090_scan/bench.cu:175-179
    return ("%12s | %10s %10s | %10s %10s\n%s" % ("Size", "CUB (ms)", "CUB (GB/s)", "Ours (ms)", "Ours (GB/s)", "-" * 62))


def scan_row(n: int, lib_ms: float, lib_gbps: float, ours_ms: float, ours_gbps: float) -> str:
    # evals/4090_scan/bench.cu:261-262
    return "%12d | %10.4f %10.2f | %10.4f %10.2f" % (n, lib_ms, lib_gbps, ours_ms, ours_gbps)


# ----------------------------------------------------------------- timing --

def _events_ms(fn, repeats: int) -> float:
    import torch
    beg, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    beg.record()
    for _ in range(repeats):
        fn()
    end.record()
    torch.cuda.synchronize()
    return beg.elapsed_time(end)


def _best_wall_ms(fn, target_ms: float) -> float:
    """benchmark_ms of evals/4090_scan/scan_harness.cuh:84-100: best of repeated (launch + sync)."""
    import torch
    best, elapsed = float("inf"), 0.0
    while elapsed < target_ms:
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t0) * 1e3
        elapsed += ms
        best = min(best, ms)
    return best


# ----------------------------------------------------------------- sweeps --

def _ok(rc: int) -> None:
    if rc != 0:
        raise RuntimeError(f"a vendor-library call failed with code {rc}")


def sweep_sgemm(out=sys.stdout, sizes=SGEMM_SIZES, repeats: int = 10) -> None:
    import torch
    from . import _lib
    lib, vendor = _lib.load(), _lib.load_vendor()
    stream = torch.cuda.current_stream().cuda_stream
    alpha, beta = 0.5, 3.0
    top = max(sizes)
    A = torch.rand((top, top), device="cuda") * 2 - 1
    B = torch.rand((top, top), device="cuda") * 2 - 1
    C = torch.rand((top, top), device="cuda") * 2 - 1
    print("\n====================================\nStarting Performance Sweep\n====================================", file=out)
    for n in sizes:
        a, b = A.flatten()[: n * n].view(n, n), B.flatten()[: n * n].view(n, n)
        c = C.flatten()[: n * n].view(n, n).clone()
        flops = 2.0 * n * n * n
        print(f"\n====================================\nSize: {n}x{n}x{n}\n====================================", file=out)
        print("\n[cuBLAS FP32]", file=out)  # slot of the vendor BLAS: rocblas_sgemm, called as runner.cu:124-132 calls cuBLAS
        ref = c.clone()
        vend = lambda: vendor.vendor_sgemm(n, n, n, alpha, a.data_ptr(), b.data_ptr(), beta, ref.data_ptr(), stream)
        _ok(vend())
        ms = _events_ms(vend, repeats)
        print(sgemm_line(ms / 1e3 / repeats, repeats * flops * 1e-9 / (ms / 1e3), n), file=out)
        for k in (1, 2, 3, 4, 5):
            print(f"\n[My Kernel {k}]", file=out)
            c.copy_(C.flatten()[: n * n].view(n, n))
            fn = lambda: lib.prism_run_my_kernel(k, n, n, n, alpha, a.data_ptr(), b.data_ptr(), beta, c.data_ptr())
            fn()
            ms = _events_ms(fn, repeats)
            print(sgemm_line(ms / 1e3 / repeats, repeats * flops * 1e-9 / (ms / 1e3), n), file=out)
        out.flush()


def sweep_scan(out=sys.stdout, log2_sizes=SCAN_LOG2_SIZES, target_ms: float = 500.0) -> None:
    import ctypes

    import torch
    from . import _lib
    lib, vendor_lib = _lib.load(), _lib.load_vendor()
    top = 1 << max(log2_sizes)
    x = torch.randint(0, 101, (top,), dtype=torch.int32, device="cuda")  # U{0..100}, scan_harness.cuh:172
    work = torch.empty_like(x)
    ws = torch.empty(lib.prism_scan_workspace_bytes(top), dtype=torch.uint8, device="cuda")
    # hipcub::DeviceScan::InclusiveSum with its temporary storage allocated once, outside the timed region
    # (evals/4090_scan/bench.cu:96-116); it scans out of place, from the pristine input into the work buffer
    need = ctypes.c_size_t(0)
    _ok(vendor_lib.vendor_scan_temp_bytes(top, ctypes.byref(need)))
    temp = torch.empty(max(need.value, 16), dtype=torch.uint8, device="cuda")
    print(scan_header(), file=out)
    for p in log2_sizes:
        n = 1 << p
        xin, buf = x[:n], work[:n]
        # the reference scans in place and restores the input outside the timed region
        def ours():
            lib.prism_launch_scan(n, buf.data_ptr(), ws.data_ptr())
        def vendor():
            _ok(vendor_lib.vendor_scan_inclusive_sum(xin.data_ptr(), buf.data_ptr(), n, temp.data_ptr(), temp.numel(), None))
        results = []
        for fn in (vendor, ours):
            best, elapsed = float("inf"), 0.0
            while elapsed < target_ms:
                buf.copy_(xin)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                fn()
                torch.cuda.synchronize()
                ms = (time.perf_counter() - t0) * 1e3
                elapsed += max(ms, 0.05)
                best = min(best, ms)
            results.append(best)
        bytes_ = n * 4 * 2
        print(scan_row(n, results[0], bytes_ / results[0] / 1e6, results[1], bytes_ / results[1] / 1e6), file=out)
        out.flush()
    print("", file=out)


def sweep_h100(out=sys.stdout, sizes=H100_SIZES, repeats: int = 8) -> None:
    import torch
    from . import _lib
    lib, vendor = _lib.load(), _lib.load_vendor()
    for n in sizes:
        A = torch.randn((n, n), device="cuda").to(torch.bfloat16)
        B = torch.randn((n, n), device="cuda").to(torch.bfloat16)
        Cc = torch.empty((n, n), dtype=torch.bfloat16, device="cuda")  # column-major M x N, as the reference
        flops = 2.0 * n * n * n
        fn = lambda: lib.prism_runmyh100(n, n, n, A.data_ptr(), B.data_ptr(), Cc.data_ptr(), None)
        # hipBLASLt, same operands and the same bf16 column-major result as the harness asks of cuBLAS (main.cu:64-73)
        Cv = torch.empty_like(Cc)
        vend = lambda: vendor.vendor_gemm_bf16_colmajor(n, n, n, A.data_ptr(), B.data_ptr(), Cv.data_ptr(), None)
        # The harness's order (main.cu:122-167): the library once, the kernel once, the two results compared, then
        # the kernel's timed launches, then the library's. The harness allows 0.1 absolute; here that, or one rounding
        # step of bf16 where a step is larger (from |C| = 16 up: two correct roundings of sums that differ in their last
        # fp32 bits may be a step apart).
        _ok(vend())
        _ok(fn())
        torch.cuda.synchronize()
        worst = 0.0
        for r0 in range(0, n, 2048):
            a, b = Cc[r0:r0 + 2048].float(), Cv[r0:r0 + 2048].float()
            worst = max(worst, float(((a - b).abs() - (2.0 ** -7 * torch.maximum(a.abs(), b.abs())).clamp(min=0.1)).max()))
        print("Passed correctness verification!" if worst <= 0.0 else
              f"Failed to pass correctness verification against hipBLASLt (beyond 0.1 and one bf16 step by {worst:g}).", file=out)
        ms = _events_ms(fn, repeats)
        print(h100_line("Kernel:", ms / 1e3 / repeats, repeats * flops * 1e-9 / ms, n), file=out)
        ms = _events_ms(vend, repeats)
        print(h100_line("cuBLAS:", ms / 1e3 / repeats, repeats * flops * 1e-9 / ms, n) + "\n", file=out)
        out.flush()
        del A, B, Cc, Cv


def sweep_generated(out=sys.stdout, sgemm_sizes=SGEMM_SIZES, scan_log2_sizes=SCAN_LOG2_SIZES, h100_sizes=H100_SIZES,
                    repeats: int = 10, target_ms: float = 500.0) -> None:
    """The three sweeps over kernels generated from the example programs."""
    import ctypes
    import tempfile

    import torch

    from . import _lib, examples, hipgen
    examples.load()
    built = {}
    vendor_lib = _lib.load_vendor()

    def kernel(name):
        if name not in built:
            _, block_size, template = examples.KERNELS[name]
            lib = hipgen.build(name, out_dir=tempfile.mkdtemp(prefix="prism_eval_"), block_size=block_size, template=template)
            built[name] = getattr(lib, f"{name}_launch")
        return built[name]

    sgemm_args = [ctypes.c_int] * 3 + [ctypes.c_float, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float, ctypes.c_void_p,
                                       ctypes.c_int, ctypes.c_uint, ctypes.c_void_p]
    # "My Kernel" k -> (program, smallest size it takes, last integer argument, number of workgroups)
    steps = {1: ("naive_sgemm", 1, lambda n: 256, lambda n: (n * n + 255) // 256),
             2: ("remapped_sgemm", 1, lambda n: (n + 31) // 32, lambda n: ((n + 31) // 32) ** 2),
             3: ("tiled_sgemm", 32, lambda n: n // 32, lambda n: (n // 32) ** 2),
             4: ("vector_tile_sgemm", 128, lambda n: n // 128, lambda n: (n // 128) ** 2),
             5: ("handed_over_sgemm", 1024, lambda n: n // 256, lambda n: (n // 128) * (n // 256))}
    # from 4096 up kernel 5 is the program in which every wavefront loads and multiplies (256 x 256 tiles)
    big5 = ("pipelined_sgemm", 4096, lambda n: n // 256, lambda n: (n // 256) ** 2)
    alpha, beta = 0.5, 3.0
    top = max(sgemm_sizes)
    A = torch.rand((top, top), device="cuda") * 2 - 1
    B = torch.rand((top, top), device="cuda") * 2 - 1
    C = torch.rand((top, top), device="cuda") * 2 - 1
    print("\n====================================\nStarting Performance Sweep\n====================================", file=out)
    for n in sgemm_sizes:
        a, b = A.flatten()[: n * n].view(n, n), B.flatten()[: n * n].view(n, n)
        c = C.flatten()[: n * n].view(n, n).clone()
        flops = 2.0 * n * n * n
        print(f"\n====================================\nSize: {n}x{n}x{n}\n====================================", file=out)
        print("\n[cuBLAS FP32]", file=out)
        ref = c.clone()
        vend = lambda: vendor_lib.vendor_sgemm(n, n, n, alpha, a.data_ptr(), b.data_ptr(), beta, ref.data_ptr(), None)
        _ok(vend())
        ms = _events_ms(vend, repeats)
        print(sgemm_line(ms / 1e3 / repeats, repeats * flops * 1e-9 / (ms / 1e3), n), file=out)
        for k, (name, smallest, last, blocks) in steps.items():
            if k == 5 and n >= big5[1] and n % 2048 == 0:
                name, smallest, last, blocks = big5
            if n < smallest:
                continue
            launch = kernel(name)
            launch.argtypes = sgemm_args
            print(f"\n[My Kernel {k}]", file=out)
            c.copy_(C.flatten()[: n * n].view(n, n))
            fn = lambda: launch(n, n, n, alpha, a.data_ptr(), b.data_ptr(), beta, c.data_ptr(), last(n), blocks(n), None)
            if fn() != 0:
                raise RuntimeError(f"{name} failed to launch at {n}")
            ms = _events_ms(fn, repeats)
            print(sgemm_line(ms / 1e3 / repeats, repeats * flops * 1e-9 / (ms / 1e3), n), file=out)
        out.flush()
    del A, B, C

    scan = kernel("lookback_scan_striped")
    scan.argtypes = [ctypes.c_void_p] * 4 + [ctypes.c_int, ctypes.c_uint, ctypes.c_void_p]
    top = 1 << max(scan_log2_sizes)
    x = torch.randint(0, 101, (top,), dtype=torch.int32, device="cuda")
    work = torch.empty_like(x)
    counter = torch.zeros(1, dtype=torch.int32, device="cuda")
    status = torch.zeros(top // 65536, dtype=torch.int64, device="cuda")
    need = ctypes.c_size_t(0)
    _ok(vendor_lib.vendor_scan_temp_bytes(top, ctypes.byref(need)))
    temp = torch.empty(max(need.value, 16), dtype=torch.uint8, device="cuda")
    print("\n" + scan_header(), file=out)
    for p in scan_log2_sizes:
        n = 1 << p
        xin, buf = x[:n], work[:n]

        def ours():  # the two clearing fills are timed, as the reference's two memsets are
            counter.zero_()
            status[: n // 65536].zero_()
            if scan(xin.data_ptr(), buf.data_ptr(), counter.data_ptr(), status.data_ptr(), 1 << 22, n // 65536, None) != 0:
                raise RuntimeError("lookback_scan_striped failed to launch")

        def vendor():
            _ok(vendor_lib.vendor_scan_inclusive_sum(xin.data_ptr(), buf.data_ptr(), n, temp.data_ptr(), temp.numel(), None))
        results = [_best_wall_ms(fn, target_ms) for fn in (vendor, ours)]
        bytes_ = n * 4 * 2
        print(scan_row(n, results[0], bytes_ / results[0] / 1e6, results[1], bytes_ / results[1] / 1e6), file=out)
        out.flush()
    print("", file=out)
    del x, work

    for n in h100_sizes:
        # 256 x 256 tiles with every wavefront loading and multiplying from 4096 up, the producer / consumer
        # kernel on 128 x 256 tiles below (twice the workgroups)
        name, rows = ("pipelined_gemm_bf16", 256) if n >= 4096 and n % 2048 == 0 else ("handed_over_gemm_big", 128)
        gemm = kernel(name)
        gemm.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_int] * 4 + [ctypes.c_uint, ctypes.c_void_p]
        P = torch.randn((n, n), device="cuda").to(torch.bfloat16)
        Q = torch.randn((n, n), device="cuda").to(torch.bfloat16)
        D = torch.empty((n, n), dtype=torch.float32, device="cuda")
        flops = 2.0 * n * n * n
        fn = lambda: gemm(P.data_ptr(), Q.data_ptr(), D.data_ptr(), n, n, n // rows, n // 256, (n // rows) * (n // 256), None)
        if fn() != 0:
            raise RuntimeError(f"{name} failed to launch at {n}")
        ms = _events_ms(fn, 8)
        print(h100_line("Kernel:", ms / 1e3 / 8, 8 * flops * 1e-9 / ms, n), file=out)
        vend = lambda: vendor_lib.vendor_gemm_bf16_f32(n, n, n, P.data_ptr(), Q.data_ptr(), D.data_ptr(), None)
        _ok(vend())
        ms = _events_ms(vend, 8)
        print(h100_line("cuBLAS:", ms / 1e3 / 8, 8 * flops * 1e-9 / ms, n) + "\n", file=out)
        out.flush()
        del P, Q, D


def main(argv=None) -> int:
    which = [a for a in (argv if argv is not None else sys.argv[1:])] or ["sgemm", "scan", "h100"]
    for w in which:
        if w == "sgemm":
            sweep_sgemm()
        elif w == "scan":
            sweep_scan()
        elif w == "h100":
            sweep_h100()
        elif w == "generated":
            sweep_generated()
        else:
            print(f"unknown sweep {w!r}; expected sgemm, scan, h100 or generated", file=sys.stderr)
            return 2
    return 0


if __name__ == "__main__":
    sys.exit(main())
