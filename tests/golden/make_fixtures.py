"""Writes tests/golden/path_fixtures.npz: small seeded inputs and expected outputs
for every operation on the path.

The reference tree holds no numeric golden vectors for this path (its scan test
generates data at run time and its GEMM checks compare against cuBLAS), so the
expected outputs here come from the CPU oracle (oracle/prism_oracle.c), after the
oracle itself has been pinned by tests/test_oracle.py. Run from the repo root:

    python tests/golden/make_fixtures.py
"""
import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))

import oracle as o  # noqa: E402


def main() -> None:
    rng = np.random.default_rng(20251125)
    fx = {}

    # add_m: BASELINE distribution plus int32 extremes (wrap-around on both ends).
    x = rng.integers(-2**20, 2**20, 1003, dtype=np.int32)
    x[:6] = np.array([2**31 - 1, 2**31 - 7, 2**31 - 8, -2**31, -1, 0], dtype=np.int32)
    fx["add_m_x"] = x
    fx["add_m_m"] = np.array([7, -9, 2**31 - 1], dtype=np.int64)
    fx["add_m_y"] = np.stack([o.add_m(x, int(m)) for m in fx["add_m_m"]])

    # scan: BASELINE distribution, ragged length that spans several tiles of any size <= 16384.
    xs = rng.integers(-1000, 1001, 40001, dtype=np.int32)
    fx["scan_x"] = xs
    fx["scan_out"] = o.scan_cpu(xs)
    # scan: the reference's own distribution and smallest two test sizes (uint32, U{0..100}).
    xu = rng.integers(0, 101, 32768, dtype=np.uint32)
    fx["scan_ref_x"] = xu
    fx["scan_ref_out"] = o.scan_cpu(xu)
    # scan: values that overflow int32 many times over.
    xw = rng.integers(2**31 - 1000, 2**31 - 1, 5000, dtype=np.int64).astype(np.int32)
    fx["scan_wrap_x"] = xw
    fx["scan_wrap_out"] = o.scan_cpu(xw)

    # sgemm: ragged shape, the reference harness's alpha/beta (evals/4090_sgemm/main.cu:48).
    M, N, K = 33, 47, 29
    A, B, Cm = o.gen_sgemm(M, N, K, seed=7)
    fx["sgemm_A"], fx["sgemm_B"], fx["sgemm_C"] = A, B, Cm
    fx["sgemm_alpha_beta"] = np.array([0.5, 3.0], dtype=np.float32)
    fx["sgemm_out_fma"] = o.sgemm_fma(0.5, A, B, 3.0, Cm)
    fx["sgemm_out_f64"] = o.sgemm_f64(0.5, A, B, 3.0, Cm)

    # bf16 gemm: ragged shape, K not a multiple of 8.
    A16, B16 = o.gen_gemm_bf16(40, 24, 75, seed=11)
    fx["bf16_A"], fx["bf16_B"] = A16, B16
    fx["bf16_D_f64"] = o.gemm_bf16_f64(A16, B16)

    out = ROOT / "tests" / "golden" / "path_fixtures.npz"
    np.savez_compressed(out, **fx)
    print(out, out.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
