"""C-ABI checks that need no GPU: the library loads, exports every function the
header declares, and its host-side argument checks behave as documented."""
import ctypes as C
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
HEADER = ROOT / "include" / "prism_amd.h"


def declared_functions():
    text = HEADER.read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(prism_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    from prism_amd import _lib
    return _lib.load()


def test_header_lists_the_expected_entry_points():
    names = declared_functions()
    for must in ("prism_add_m", "prism_scan_i32", "prism_scan_i32_ex", "prism_scan_workspace_bytes",
                 "prism_scan_workspace_init", "prism_scan_status", "prism_launch_scan",
                 "prism_sgemm", "prism_run_my_kernel", "prism_gemm_bf16", "prism_runmyh100"):
        assert must in names


def test_library_exports_every_declared_symbol(lib):
    from prism_amd import _lib
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} declared in prism_amd.h but not exported"
        assert name in _lib.SIGNATURES, f"{name} has no ctypes signature"
    assert set(_lib.SIGNATURES) == set(declared_functions())


def test_every_declaration_cites_the_reference():
    text = HEADER.read_text()
    # each entry point's comment names the reference file it replaces
    for name, cite in [("prism_add_m", "add_m_thread.py"), ("prism_scan_workspace_bytes", "4090_scan/main.cu"),
                       ("prism_scan_i32", "scan.py"), ("prism_scan_i32_ex", "lookback_to_prev_blocks.cu"),
                       ("prism_scan_workspace_init", "4090_scan/main.cu:81-82"), ("prism_scan_i64", "scan_harness.cuh:30-36"),
                       ("prism_segmented_scan_i32", "scan.py:106-227"), ("prism_scan_exclusive_i32", "scan.py:174-193"),
                       ("prism_scan_max_i32", "scan.py:106-173"), ("prism_scan_min_i32", "scan.py:106-173"),
                       ("prism_launch_scan", "4090_scan/main.cu"),
                       ("prism_sgemm", "runner.cu"), ("prism_run_my_kernel", "runner.cu"),
                       ("prism_sgemm_ws", "evals/4090_sgemm/runner.cu:191-243"),
                       ("prism_gemm_bf16", "h100_matmul.py"), ("prism_runmyh100", "utils.cuh")]:
        decl = text.index(name + "(")
        comment = text.rfind("/*", 0, decl)
        assert cite in text[comment:decl], f"{name}: no citation of {cite}"


def test_version_and_error_string(lib):
    assert lib.prism_version().decode().count(".") == 2
    assert isinstance(lib.prism_last_error_string(), bytes)


def test_argument_checks_run_before_any_gpu_work(lib):
    # unknown kernel numbers: the reference throws std::invalid_argument (runner.cu:265)
    for bad in (0, 6, -1, 99):
        assert lib.prism_run_my_kernel(bad, 4, 4, 4, 1.0, None, None, 0.0, None) == 1
        assert b"Unknown my_kernel number" in lib.prism_last_error_string()
    assert lib.prism_sgemm(7, 4, 4, 4, 1.0, None, None, 0.0, None, None) == 1
    assert lib.prism_sgemm(5, -1, 4, 4, 1.0, None, None, 0.0, None, None) == 1
    assert lib.prism_sgemm(5, 4, 4, 4, 1.0, None, None, 0.0, None, None) == 1  # null matrices
    # the workspace form checks the same things before it looks at the workspace
    assert lib.prism_sgemm_ws(7, 4, 4, 4, 1.0, None, None, 0.0, None, None, 0, None) == 1
    assert b"unknown kernel number" in lib.prism_last_error_string()
    assert lib.prism_sgemm_ws(5, 128, 4096, -4096, 1.0, None, None, 0.0, None, None, 0, None) == 1
    assert lib.prism_sgemm_ws(5, 128, 4096, 4096, 1.0, None, None, 0.0, None, None, 0, None) == 1
    assert b"null matrix pointer" in lib.prism_last_error_string()
    # the workspace form checks like prism_sgemm; the size query needs no device (256 CUs assumed without one)
    assert lib.prism_sgemm_ws(7, 4, 4, 4, 1.0, None, None, 0.0, None, None, 0, None) == 1
    assert lib.prism_sgemm_ws(5, 4, 4, 4, 1.0, None, None, 0.0, None, None, 0, None) == 1
    assert lib.prism_sgemm_ws(5, 0, 4, 4, 1.0, None, None, 0.0, None, None, 0, None) == 0
    assert lib.prism_sgemm_workspace_bytes(128, 4096, 4096) % (128 * 4096 * 4) == 0
    assert lib.prism_sgemm_workspace_bytes(128, 4096, 4096) >= 2 * 128 * 4096 * 4      # a skinny product is cut
    for whole_chip in ((8192, 8192, 8192), (4096, 4096, 128), (128, 4096, 100), (100, 4096, 4096), (0, 4096, 4096), (-1, 4, 4)):
        assert lib.prism_sgemm_workspace_bytes(*whole_chip) == 0
    # empty problems succeed without touching a device
    assert lib.prism_sgemm(5, 0, 4, 4, 1.0, None, None, 0.0, None, None) == 0
    assert lib.prism_add_m(None, None, 7, 0, None) == 0
    assert lib.prism_scan_i32(None, None, 0, None, 0, None) == 0
    assert lib.prism_gemm_bf16(0, 8, 8, None, None, None, None) == 0
    assert lib.prism_add_m(None, None, 7, 5, None) == 1
    assert lib.prism_gemm_bf16(8, 8, -8, None, None, None, None) == 1
    # misaligned and overlapping buffers are rejected
    assert lib.prism_add_m(0x1002, 0x2000, 7, 4, None) == 1
    assert lib.prism_add_m(0x1000, 0x1008, 7, 4, None) == 1
    assert lib.prism_scan_i32(0x1000, 0x1004, 16, 0x9000, 1 << 20, None) == 1
    # workspace too small
    need = lib.prism_scan_workspace_bytes(1 << 20)
    assert lib.prism_scan_i32(0x100000, 0x100000, 1 << 20, 0x9000, need - 1, None) == 1
    assert b"workspace" in lib.prism_last_error_string()
    # the explicit form: unknown flag bits, flag combinations that do not exist, workspace alignment
    assert lib.prism_scan_i32_ex(0x100000, 0x100000, 1 << 20, 0x9000, need, 0x40, -1, None) == 1
    assert b"flag" in lib.prism_last_error_string()
    assert lib.prism_scan_i32_ex(0x100000, 0x100000, 1 << 20, 0x9000, need, 0x30, -1, None) == 1
    assert lib.prism_scan_i32_ex(0x100000, 0x100000, 1 << 20, 0x9000, need, 0x10 | 1, -1, None) == 1
    assert lib.prism_scan_i32_ex(0x100000, 0x100000, 1 << 20, 0x9008, need, 0, -1, None) == 1
    assert lib.prism_scan_i32_ex(None, None, 0, None, 0, 3, 0, None) == 0
    assert lib.prism_scan_workspace_init(None, 4096, None) == 1
    assert lib.prism_scan_workspace_init(0x9000, 8, None) == 1
    assert lib.prism_scan_workspace_init(0x9004, 4096, None) == 1


def test_scan_workspace_size(lib):
    sizes = [lib.prism_scan_workspace_bytes(n) for n in (0, 1, 4096, 4097, 1 << 20, 1 << 30)]
    assert all(s > 0 and s % 16 == 0 for s in sizes)
    assert sizes == sorted(sizes)
    # a header plus the reference's 16 bytes per 16384 elements (main.cu:63-66)
    assert sizes[-1] == 256 + ((1 << 30) // 16384 + 1) * 16 and sizes[0] == 256 + 16


@pytest.mark.parametrize("tiles", [(1, 1), (1, 9), (7, 1), (8, 8), (64, 64), (3, 5), (33, 17), (64, 33), (5, 129)])
def test_tile_map_is_a_bijection(lib, tiles):
    tm_n, tn_n = tiles
    seen = set()
    tm, tn = C.c_int(), C.c_int()
    for wg in range(tm_n * tn_n):
        assert lib.prism_tile_coords(wg, tm_n, tn_n, C.byref(tm), C.byref(tn)) == 0
        assert 0 <= tm.value < tm_n and 0 <= tn.value < tn_n
        seen.add((tm.value, tn.value))
    assert len(seen) == tm_n * tn_n
    assert lib.prism_tile_coords(tm_n * tn_n, tm_n, tn_n, C.byref(tm), C.byref(tn)) == 1


def test_tile_map_keeps_an_xcd_on_a_compact_patch(lib):
    """Workgroups 8 apart run on the same XCD; the first 64 of them (two per CU)
    must cover a patch that shares A row-panels and B column-panels: at most 8
    distinct tile rows and 8 distinct tile columns on a 64 x 64 grid."""
    tm, tn = C.c_int(), C.c_int()
    for xcd in range(8):
        rows, cols = set(), set()
        for i in range(64):
            lib.prism_tile_coords(xcd + 8 * i, 64, 64, C.byref(tm), C.byref(tn))
            rows.add(tm.value)
            cols.add(tn.value)
        assert len(rows) <= 8 and len(cols) <= 8


def test_header_is_valid_c_and_cxx(tmp_path):
    """include/prism_amd.h must compile as plain C99 and as C++ (it is the FFI contract)."""
    import shutil
    import subprocess
    src_c = tmp_path / "t.c"
    src_c.write_text('#include "prism_amd.h"\nint main(void) { return (int)sizeof(&prism_scan_i32) == 0; }\n')
    src_cc = tmp_path / "t.cpp"
    src_cc.write_text('#include "prism_amd.h"\nint main() { return PRISM_SGEMM_WAVE_TILE == 5 ? 0 : 1; }\n')
    inc = str(ROOT / "include")
    if shutil.which("gcc"):
        subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-fsyntax-only", "-I", inc, str(src_c)], check=True)
    if shutil.which("g++"):
        subprocess.run(["g++", "-std=c++11", "-Wall", "-Werror", "-fsyntax-only", "-I", inc, str(src_cc)], check=True)
