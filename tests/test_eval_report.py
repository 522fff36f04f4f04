"""The text prism_amd.eval_report prints must be readable by the reference's plotting script.
The regular expressions below are the ones evals/plot_results.py uses (lines 24-33, 52-77, 88-105)."""
import io
import re

import pytest

from prism_amd import eval_report as er

H100_KERNEL = r'Kernel:\s+.*performance:\s+\(\s*([\d.]+)\)\s+TFLOPS.*size:\s+\((\d+)\)'
H100_VENDOR = r'cuBLAS:\s+.*performance:\s+\(\s*([\d.]+)\)\s+TFLOPS.*size:\s+\((\d+)\)'
SGEMM_PERF = r'performance:\s+\(\s*([\d.]+)\)\s+GFLOPS.*size:\s+\((\d+)\)'


def parse_scan_table(text):
    rows, in_table = [], False
    for line in text.splitlines():
        if 'Size' in line and 'CUB (GB/s)' in line:
            in_table = True
            continue
        if in_table and line.strip().startswith('---'):
            continue
        if in_table and line.strip():
            parts = re.split(r'\s*\|\s*', line.strip())
            rows.append((int(parts[0]), float(parts[1].split()[1]), float(parts[2].split()[1])))
        elif in_table:
            in_table = False
    return rows


def parse_sgemm(text):
    out, size, kernel, perf = {}, None, None, False
    for line in text.splitlines():
        if 'Starting Performance Sweep' in line:
            perf = True
        if not perf:
            continue
        m = re.match(r'Size:\s+(\d+)x(\d+)x(\d+)', line.strip())
        if m:
            size = int(m.group(1))
        if re.match(r'\[cuBLAS FP32\]', line.strip()):
            kernel = 'vendor'
        m = re.match(r'\[My Kernel (\d+)\]', line.strip())
        if m:
            kernel = int(m.group(1))
        m = re.search(SGEMM_PERF, line)
        if m and kernel is not None:
            out.setdefault(kernel, []).append((size, float(m.group(1)), int(m.group(2))))
            kernel = None
    return out


def test_line_formats_match_the_reference_parsers():
    m = re.search(SGEMM_PERF, er.sgemm_line(0.008403, 130858.4, 8192))
    assert m and float(m.group(1)) == 130858.4 and int(m.group(2)) == 8192
    m = re.search(H100_KERNEL, er.h100_line("Kernel:", 0.000880, 1250.0, 8192))
    assert m and float(m.group(1)) == 1250.0 and int(m.group(2)) == 8192
    m = re.search(H100_VENDOR, er.h100_line("cuBLAS:", 0.000830, 1324.5, 8192))
    assert m and float(m.group(1)) == 1324.5
    table = er.scan_header() + "\n" + er.scan_row(1 << 30, 1.9, 4500.12, 1.6, 5368.71) + "\n\n"
    assert parse_scan_table(table) == [(1 << 30, 4500.12, 5368.71)]


@pytest.mark.gpu
def test_sweeps_produce_parseable_reports():
    buf = io.StringIO()
    er.sweep_sgemm(buf, sizes=(256, 512), repeats=3)
    parsed = parse_sgemm(buf.getvalue())
    assert sorted(parsed, key=str) == [1, 2, 3, 4, 5, 'vendor']
    for rows in parsed.values():
        assert [r[0] for r in rows] == [256, 512] and all(r[1] > 0 for r in rows)

    buf = io.StringIO()
    er.sweep_scan(buf, log2_sizes=(20, 22), target_ms=20.0)
    rows = parse_scan_table(buf.getvalue())
    assert [r[0] for r in rows] == [1 << 20, 1 << 22] and all(r[1] > 0 and r[2] > 0 for r in rows)

    buf = io.StringIO()
    er.sweep_h100(buf, sizes=(2048, 4352), repeats=3)
    text = buf.getvalue()
    assert re.search(H100_KERNEL, text) and re.search(H100_VENDOR, text)
    # the harness's comparison with the vendor library (evals/h100_bench/main.cu:122-135), once per size
    assert text.count("Passed correctness verification!") == 2 and "Failed" not in text


@pytest.mark.gpu
def test_sweeps_over_generated_kernels_produce_parseable_reports():
    """The same three formats from kernels generated out of the example programs (compiled on the spot)."""
    buf = io.StringIO()
    er.sweep_generated(buf, sgemm_sizes=(256, 1024), scan_log2_sizes=(20, 22), h100_sizes=(1024,), repeats=2, target_ms=20.0)
    text = buf.getvalue()
    parsed = parse_sgemm(text)
    assert sorted(parsed, key=str) == [1, 2, 3, 4, 5, 'vendor']
    assert [r[0] for r in parsed[1]] == [256, 1024] and [r[0] for r in parsed[5]] == [1024]   # the last step starts at 1024
    assert all(r[1] > 0 for rows in parsed.values() for r in rows)
    rows = parse_scan_table(text)
    assert [r[0] for r in rows] == [1 << 20, 1 << 22] and all(r[1] > 0 and r[2] > 0 for r in rows)
    assert re.search(H100_KERNEL, text) and re.search(H100_VENDOR, text)


def test_vendor_baseline_library_builds_and_exports_its_entry_points():
    """hipCUB, rocBLAS and hipBLASLt behind plain C entry points: a library of its own, every symbol typed."""
    from prism_amd import _lib
    lib = _lib.load_vendor()
    for name in _lib.VENDOR_SIGNATURES:
        assert hasattr(lib, name)


@pytest.mark.gpu
def test_vendor_baselines_compute_what_the_sweeps_compare_with(oracle):
    """The vendor-library calls are handed operands in this repository's layouts (row-major fp32; bf16 A M x K and
    B N x K; the harness's column-major bf16 result): their results must be the same products the library's own
    kernels are checked against, or the comparison lines of the sweeps would time something else."""
    import ctypes

    import numpy as np
    import torch
    from prism_amd import _lib
    v = _lib.load_vendor()
    dev = "cuda:0"
    # scan: exact
    n = (1 << 22) + 1234
    x = oracle.gen_scan(n, seed=1)
    xd = torch.from_numpy(x).to(dev)
    out = torch.empty_like(xd)
    need = ctypes.c_size_t(0)
    assert v.vendor_scan_temp_bytes(n, ctypes.byref(need)) == 0
    temp = torch.empty(max(need.value, 16), dtype=torch.uint8, device=dev)
    assert v.vendor_scan_inclusive_sum(xd.data_ptr(), out.data_ptr(), n, temp.data_ptr(), temp.numel(), None) == 0
    torch.cuda.synchronize()
    assert np.array_equal(out.cpu().numpy(), oracle.scan_cpu(x))
    # sgemm: a ragged, non-square shape shows a transposed operand or a swapped dimension
    M, N, K = 200, 328, 136
    A, B, Cm = oracle.gen_sgemm(M, N, K, seed=2)
    c = torch.from_numpy(Cm).to(dev)
    assert v.vendor_sgemm(M, N, K, 0.5, torch.from_numpy(A).to(dev).data_ptr(), torch.from_numpy(B).to(dev).data_ptr(), 3.0,
                          c.data_ptr(), None) == 0
    torch.cuda.synchronize()
    assert np.max(np.abs(c.cpu().numpy() - oracle.sgemm_f64(0.5, A, B, 3.0, Cm))) <= oracle.sgemm_tolerance(K, A, B) + 3.0 * 2**-22
    # bf16: fp32 row-major result and bf16 column-major result
    M, N, K = 192, 320, 136
    A16, B16 = oracle.gen_gemm_bf16(M, N, K, seed=3)
    a = torch.from_numpy(A16.view(np.int16)).to(dev)
    b = torch.from_numpy(B16.view(np.int16)).to(dev)
    ref = oracle.gemm_bf16_f64(A16, B16)
    d = torch.empty((M, N), dtype=torch.float32, device=dev)
    assert v.vendor_gemm_bf16_f32(M, N, K, a.data_ptr(), b.data_ptr(), d.data_ptr(), None) == 0
    cc = torch.empty(N * M, dtype=torch.int16, device=dev)
    assert v.vendor_gemm_bf16_colmajor(M, N, K, a.data_ptr(), b.data_ptr(), cc.data_ptr(), None) == 0
    torch.cuda.synchronize()
    assert np.max(np.abs(d.cpu().numpy() - ref)) <= 1e-3 * np.abs(ref).max()
    got = oracle.bf16_to_f32(cc.cpu().numpy().view(np.uint16)).reshape(N, M).T
    assert np.max(np.abs(got - ref)) <= 2.0**-8 * np.abs(ref).max()
