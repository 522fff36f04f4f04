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
    er.sweep_h100(buf, sizes=(2048,), repeats=3)
    text = buf.getvalue()
    assert re.search(H100_KERNEL, text) and re.search(H100_VENDOR, text)


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
