"""The double-buffered GEMMs in which every wavefront loads and multiplies (prism_amd/examples/pipelined.py).

CPU: the programs pass the perspective rules, and the access analysis gives them one workgroup barrier per K
tile (one in front of the loop, one in front of the refill of the first stage, one at the end of the loop body;
the refill sits in an `if`, so its barrier stands in front of the `if`). GPU: both kernels against the fp64
oracles (kernel 5's tolerance for fp32, 1e-3 of the largest |element| for bf16).
"""
import ctypes

import numpy as np
import pytest

from prism_amd import hipgen
from prism_amd.examples import pipelined  # noqa: F401  (defines the kernels)
from prism_amd.hipgen import generate
from prism_amd.hipgen_check import check


def lines(text):
    return [ln.strip() for ln in text.splitlines()]


@pytest.mark.parametrize("name,step,fill,multiply", [("pipelined_sgemm", 64, "fill_stage_f32", "multiply_stage_f32"),
                                                    ("pipelined_gemm_bf16", 128, "fill_stage_bf16", "multiply_stage_bf16")])
def test_one_barrier_per_k_tile(name, step, fill, multiply):
    for fn in (name, fill, multiply):
        check(fn)
    got = lines(generate(name))
    loop = got.index(f"for (int k0 = 0; k0 < K; k0 += {step}) {{")
    def kind(ln):
        if ln.startswith(fill + "("):
            return "fill"
        if ln.startswith(multiply + "("):
            return "multiply"
        if ln == "__syncthreads();":
            return "barrier"
        if ln.startswith("if (((k0 +"):
            return "if"
        if ln.startswith("for (int k0"):
            return "loop"
        return None
    order = [kind(ln) for ln in got if kind(ln)]
    # the bf16 program refills its first stage unconditionally (a branch would end the stretch of code its
    # scheduling groups order), the fp32 one under `if k0 + 64 < K`
    refill = ["fill"] if name == "pipelined_gemm_bf16" else ["if", "fill"]
    assert order == ["fill", "barrier", "loop", "fill", "multiply", "barrier", *refill, "multiply", "barrier"]
    if name == "pipelined_gemm_bf16":   # the scheduling groups stand between a multiplication and the barrier behind it
        at = [n for n, ln in enumerate(got) if ln.startswith(multiply + "(")]
        assert all(got[n + 1] == "__builtin_amdgcn_sched_group_barrier(0x100, 5, 0);" for n in at)
        assert sum(ln.startswith("__builtin_amdgcn_sched_group_barrier(") for ln in got) == 2 * 10
    assert got.index("__syncthreads();") < loop                       # the first one stands in front of the loop
    assert got.count("__syncthreads();") == 3                         # and the write-back needs none
    assert "__hip_atomic" not in "\n".join(got)                       # no hand-over counters: nobody splits


@pytest.fixture(scope="module")
def built_sgemm(tmp_path_factory):
    return hipgen.build("pipelined_sgemm", out_dir=str(tmp_path_factory.mktemp("hipgen_pipelined_sgemm")), block_size=1024)


@pytest.fixture(scope="module")
def built_bf16(tmp_path_factory):
    return hipgen.build("pipelined_gemm_bf16", out_dir=str(tmp_path_factory.mktemp("hipgen_pipelined_bf16")), block_size=512)


def test_launchers_compile_for_gfx950(built_sgemm, built_bf16):
    assert hasattr(built_sgemm, "pipelined_sgemm_launch") and hasattr(built_bf16, "pipelined_gemm_bf16_launch")


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(2048, 256, 64), (2048, 768, 960), (4096, 1024, 2048)])
def test_pipelined_sgemm_against_the_oracle(built_sgemm, oracle, shape):
    import torch
    M, N, K = shape
    fn = built_sgemm.pipelined_sgemm_launch
    fn.argtypes = [ctypes.c_int] * 3 + [ctypes.c_float, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float, ctypes.c_void_p,
                                       ctypes.c_int, ctypes.c_uint, ctypes.c_void_p]
    A, B, Cm = oracle.gen_sgemm(M, N, K, seed=M + N + K)
    a, b = torch.from_numpy(A).to("cuda:0"), torch.from_numpy(B).to("cuda:0")
    buf = torch.full((M * N + 128,), 777.0, dtype=torch.float32, device="cuda:0")
    c = buf[64:64 + M * N].view(M, N)
    c.copy_(torch.from_numpy(Cm))
    torch.cuda.synchronize()
    print(f"pipelined_sgemm M={M} N={N} K={K}", flush=True)
    assert fn(M, N, K, 0.5, a.data_ptr(), b.data_ptr(), 3.0, c.data_ptr(), N // 256, (M // 256) * (N // 256), None) == 0
    torch.cuda.synchronize()
    out = buf.cpu().numpy()
    assert np.all(out[:64] == 777.0) and np.all(out[64 + M * N:] == 777.0)
    want = oracle.np_sgemm_f64(0.5, A, B, 3.0, Cm)
    tol = oracle.sgemm_tolerance(K, A, B) + 3.0 * float(np.abs(Cm).max()) * 2**-22
    assert np.max(np.abs(out[64:64 + M * N].reshape(M, N) - want)) <= tol


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(2048, 256, 128), (2048, 512, 1152), (4096, 1024, 768)])
def test_pipelined_gemm_bf16_against_the_oracle(built_bf16, oracle, shape):
    import torch
    M, N, K = shape
    fn = built_bf16.pipelined_gemm_bf16_launch
    fn.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_int] * 4 + [ctypes.c_uint, ctypes.c_void_p]
    p16, q16 = oracle.gen_gemm_bf16(M, N, K, seed=M + N + K + 2)
    P = torch.from_numpy(p16.view(np.int16)).to("cuda:0")
    Q = torch.from_numpy(q16.view(np.int16)).to("cuda:0")
    buf = torch.full((M * N + 128,), 777.0, dtype=torch.float32, device="cuda:0")
    D = buf[64:64 + M * N]
    torch.cuda.synchronize()
    print(f"pipelined_gemm_bf16 M={M} N={N} K={K}", flush=True)
    assert fn(P.data_ptr(), Q.data_ptr(), D.data_ptr(), N, K, M // 256, N // 256, (M // 256) * (N // 256), None) == 0
    torch.cuda.synchronize()
    out = buf.cpu().numpy()
    assert np.all(out[:64] == 777.0) and np.all(out[64 + M * N:] == 777.0)
    ref = oracle.gemm_bf16_f64(p16, q16)
    assert np.max(np.abs(out[64:64 + M * N].reshape(M, N) - ref)) <= 1e-3 * np.abs(ref).max()
