"""Compile libprism_amd.so for gfx950 with hipcc, in-tree.

Usage: ``python -m prism_amd.build`` (or ``prism_amd.build.build()``).
The library is never built implicitly at import time on a machine that
already holds one; loading code calls :func:`ensure_built` which compiles
only when the file is missing.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_PATH = PKG_DIR / "libprism_amd.so"
SOURCES = ["capi.hip", "add_m.hip", "scan.hip", "sgemm.hip", "gemm_bf16.hip", "regroup.hip"]

# -packed-fp32-ops: keep the compiler from forming v_pk_*_f32 out of scalar
# float code; the kernels here get their fp32 throughput from MFMA instead.
HIPCC_FLAGS = [
    "-O3",
    "-std=c++17",
    "--offload-arch=gfx950",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def hipcc_path() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or add /opt/rocm/bin to PATH)")


def _run(cmd: list[str], verbose: bool) -> None:
    if verbose:
        print(" ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # The host pass does not know the packed-fp32 feature and says so; drop that line.
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)


def build(verbose: bool = False, extra_flags: list[str] | None = None, output: Path | None = None,
          sources: list[str] | None = None) -> Path:
    """Compile every kernel source into one shared library; always recompiles. The sources are compiled
    side by side (one hipcc process each) into a scratch directory and linked."""
    import tempfile
    from concurrent.futures import ThreadPoolExecutor

    out = Path(output) if output else LIB_PATH
    hipcc = hipcc_path()
    flags = [*HIPCC_FLAGS, *(extra_flags or [])]
    names = sources or SOURCES
    with tempfile.TemporaryDirectory(prefix="prism_amd_build_") as tmp:
        objs = [str(Path(tmp) / (Path(s).stem + ".o")) for s in names]
        jobs = [[hipcc, *flags, "-c", str(CSRC / s), "-o", o] for s, o in zip(names, objs)]
        with ThreadPoolExecutor(max_workers=min(len(jobs), os.cpu_count() or 1, 16)) as pool:
            list(pool.map(lambda c: _run(c, verbose), jobs))
        _run([hipcc, *flags, "-shared", "-o", str(out), *objs], verbose)
    return out


def ensure_built() -> Path:
    if not LIB_PATH.exists():
        build()
    return LIB_PATH


# The vendor libraries behind plain C entry points (hipCUB, rocBLAS, hipBLASLt called directly): the baselines of
# the evaluation sweeps. A library of its own, so that libprism_amd.so links nothing but the HIP runtime.
VENDOR_LIB_PATH = PKG_DIR / "libprism_vendor_baselines.so"


def build_vendor_baselines(verbose: bool = False) -> Path:
    _run([hipcc_path(), *HIPCC_FLAGS, "-shared", "-o", str(VENDOR_LIB_PATH), str(CSRC / "vendor" / "vendor_baselines.hip"),
          "-lrocblas", "-lhipblaslt"], verbose)
    return VENDOR_LIB_PATH


def ensure_vendor_built() -> Path:
    if not VENDOR_LIB_PATH.exists():
        build_vendor_baselines()
    return VENDOR_LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
    print(build_vendor_baselines(verbose=True))
