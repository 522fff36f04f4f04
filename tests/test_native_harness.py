"""The launcher replacements that the integration guide shows to a maintainer of the reference's harnesses, compiled
as C++ against include/prism_amd.h, linked with libprism_amd.so and run.

tests/native/harness_main.cpp is this repository's own stand-in for the three harness mains (their
correctness runs in outline: scan_harness.cuh:112-168, 4090_sgemm/main.cu:84-147, h100_bench/main.cu:123-141);
the C++ code blocks of the guide's sections 1-3 are extracted verbatim into the file it includes, so the
documentation's snippets are what is compiled and executed. Host code only (g++ against the HIP runtime API).
"""
import re
import shutil
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
ROCM = Path("/opt/rocm")


def build_harness(out_dir: Path) -> Path:
    from prism_amd.build import LIB_PATH, ensure_built
    ensure_built()
    text = (ROOT / "INTEGRATION.md").read_text()
    head = text[text.index("## 1. Scan harness"):text.index("## 4. add_m")]
    blocks = re.findall(r"```cpp\n(.*?)```", head, flags=re.S)
    assert len(blocks) == 4, "sections 1-3 of the integration guide hold four C++ blocks (section 2 has two)"
    out_dir.mkdir(parents=True, exist_ok=True)
    (out_dir / "integration_snippets.inc").write_text("\n".join(blocks))
    exe = out_dir / "native_harness"
    cmd = [shutil.which("g++") or "g++", "-std=c++17", "-O1", "-Wall", "-Werror", "-D__HIP_PLATFORM_AMD__",
           f"-I{ROCM / 'include'}", f"-I{ROOT / 'include'}", f"-I{out_dir}",
           str(ROOT / "tests" / "native" / "harness_main.cpp"), "-o", str(exe),
           f"-L{LIB_PATH.parent}", "-lprism_amd", f"-L{ROCM / 'lib'}", "-lamdhip64",
           f"-Wl,-rpath,{LIB_PATH.parent}", f"-Wl,-rpath,{ROCM / 'lib'}"]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    assert proc.returncode == 0, proc.stderr
    return exe


def test_integration_snippets_compile_and_link(tmp_path):
    exe = build_harness(tmp_path)
    assert exe.exists()


@pytest.mark.gpu
def test_integration_snippets_run(tmp_path):
    exe = build_harness(tmp_path)
    proc = subprocess.run([str(exe)], capture_output=True, text=True, timeout=110)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert proc.stdout.strip().endswith("OK")
    for must in ("scan n=16384 ok", "scan n=1048593 ok", "sgemm kernel 5 n=256 ok", "sgemm with workspace 64x256x16384 ok",
                 "h100 256x512x192 ok"):
        assert must in proc.stdout
