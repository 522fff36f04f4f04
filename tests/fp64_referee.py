"""Full-size GEMM checks: every element of a device result against an fp64 product formed on the device.

At 4096^3 .. 16384^3 the scalar CPU oracle cannot form the whole product (8192^3 is half a day of one core), so
the full-size tests and the benchmark's parity gate compare against torch's fp64 GEMM on the same GPU. That
referee is itself pinned to the oracle: `pin_sgemm_referee` / `pin_gemm_bf16_referee` recompute sampled rows
of the same device product with `oracle.sgemm_f64` / `oracle.gemm_bf16_f64` (serial fp64 loops, pinned in
tests/test_oracle.py) and return the largest deviation relative to the largest element, which the tests bound
by 1e-9 (two fp64 sums of K products of the same numbers differ by about K * 2^-53 of their magnitude).

Test infrastructure: the benchmark imports its parity gate from here; nothing under prism_amd/ does.
"""
from __future__ import annotations

import numpy as np


def _sgemm_ref_rows(alpha, A_rows, Bd, beta, C0_rows):
    """alpha * A_rows @ B + beta * C0_rows in fp64 on the device (Bd is B already in fp64)."""
    import torch
    ref = torch.matmul(A_rows.double(), Bd).mul_(alpha)
    if beta != 0:
        ref.add_(C0_rows.double(), alpha=beta)
    return ref


def sgemm_max_err_fp64(alpha, A, B, beta, C0, C, rows: int = 1024) -> float:
    """max |C - (alpha A @ B + beta C0)| over EVERY element, `rows` rows of C at a time."""
    Bd = B.double()
    worst = 0.0
    for s in range(0, A.shape[0], rows):
        ref = _sgemm_ref_rows(alpha, A[s:s + rows], Bd, beta, C0[s:s + rows])
        worst = max(worst, float((C[s:s + rows].double() - ref).abs().max()))
    return worst


def gemm_bf16_max_err_fp64(A, B, D, rows: int = 1024):
    """(max |D - A @ B^T| over every element, max |A @ B^T|); the product of the bf16 inputs in fp64 on the device."""
    import torch
    Bt = B.double().T.contiguous()
    worst, ref_max = 0.0, 0.0
    for s in range(0, A.shape[0], rows):
        ref = torch.matmul(A[s:s + rows].double(), Bt)
        worst = max(worst, float((D[s:s + rows].double() - ref).abs().max()))
        ref_max = max(ref_max, float(ref.abs().max()))
    return worst, ref_max


def sample_rows(m: int, count: int = 32, seed: int = 0) -> np.ndarray:
    """`count` distinct row numbers: the first and last row and seeded draws in between."""
    count = min(count, m)
    rng = np.random.default_rng(seed)
    picked = {0, m - 1}
    while len(picked) < count:
        picked.add(int(rng.integers(0, m)))
    return np.array(sorted(picked), dtype=np.int64)


def pin_sgemm_referee(oracle, alpha, A, B, beta, C0, count: int = 32, seed: int = 0) -> float:
    """Largest |device fp64 product - oracle.sgemm_f64| over `count` sampled rows, relative to the largest element
    of those rows. A, B, C0 are device tensors; the oracle runs on host copies of the sampled rows."""
    import torch
    rows = sample_rows(A.shape[0], count, seed)
    it = torch.from_numpy(rows).to(A.device)
    dev = _sgemm_ref_rows(alpha, A[it], B.double(), beta, C0[it]).cpu().numpy()
    want = oracle.sgemm_f64(alpha, A[it].cpu().numpy(), B.cpu().numpy(), beta, C0[it].cpu().numpy())
    return float(np.max(np.abs(dev - want)) / max(np.max(np.abs(want)), 1e-300))


def pin_gemm_bf16_referee(oracle, A, B, count: int = 32, seed: int = 0) -> float:
    """The same for the bf16 GEMM's referee: sampled rows of A @ B^T (bf16 inputs, fp64 product) against
    oracle.gemm_bf16_f64 on the 16-bit patterns."""
    import torch
    rows = sample_rows(A.shape[0], count, seed)
    it = torch.from_numpy(rows).to(A.device)
    dev = torch.matmul(A[it].double(), B.double().T.contiguous()).cpu().numpy()
    bits = lambda t: t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)
    want = oracle.gemm_bf16_f64(bits(A[it]), bits(B))
    return float(np.max(np.abs(dev - want)) / max(np.max(np.abs(want)), 1e-300))
