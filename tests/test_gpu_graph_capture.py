"""Every entry point can be recorded into a HIP graph and replayed.

The entry points only enqueue kernels on the stream they are handed (a scan leaves its workspace ready for
the next one, and the one-time workspace initialisation is a fill kernel, not a memset node), so a caller
with a launch-bound loop of small problems can capture the sequence once and replay it. The graph below chains all four kernel families; it is replayed several
times with fresh input contents and eager work and synchronisations in between, and every replay is
checked against the eager result and against the oracle.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def test_capture_and_replay_all_kernel_families(prism, oracle):
    n = (1 << 18) + 77
    M, N, K = 192, 320, 136
    x = torch.zeros(n, dtype=torch.int32, device=DEV)
    shifted = torch.empty_like(x)
    scanned = torch.empty_like(x)
    ws = prism.new_scan_workspace(n)
    A = torch.zeros((M, K), dtype=torch.float32, device=DEV)
    B = torch.zeros((K, N), dtype=torch.float32, device=DEV)
    C0 = torch.zeros((M, N), dtype=torch.float32, device=DEV)
    C = torch.empty_like(C0)
    P = torch.zeros((M, K), dtype=torch.bfloat16, device=DEV)
    Q = torch.zeros((N, K), dtype=torch.bfloat16, device=DEV)
    D = torch.empty((M, N), dtype=torch.float32, device=DEV)

    def sequence():
        prism.add_m(x, shifted, 7)
        prism.scan(shifted, scanned, ws, check=False)  # the check waits for the stream: not inside a capture
        C.copy_(C0)
        prism.sgemm(M, N, K, 1.5, A, B, 0.5, C, variant=5)
        prism.sgemm(M, N, K, 1.0, A, B, 1.0, C, variant=4)
        prism.gemm_bf16(P, Q, D)

    def load(seed):
        xs = oracle.gen_scan(n, seed=seed)
        a, b, c = oracle.gen_sgemm(M, N, K, seed=seed)
        p16, q16 = oracle.gen_gemm_bf16(M, N, K, seed=seed)
        x.copy_(torch.from_numpy(xs))
        A.copy_(torch.from_numpy(a)); B.copy_(torch.from_numpy(b)); C0.copy_(torch.from_numpy(c))
        P.copy_(torch.from_numpy(p16.view(np.int16)).view(torch.bfloat16))
        Q.copy_(torch.from_numpy(q16.view(np.int16)).view(torch.bfloat16))
        return xs, a, b, c, p16, q16

    load(0)
    side = torch.cuda.Stream()  # default priority
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        sequence()  # warm-up outside the capture (first-call work such as the device query)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        sequence()

    for seed in (1, 2, 3):
        xs, a, b, c, p16, q16 = load(seed)
        sequence()  # eager, on the current stream
        torch.cuda.synchronize()
        eager = [t.clone() for t in (scanned, C, D)]
        for t in (shifted, scanned, C, D):
            t.fill_(0)  # eager work between the replays; a replay that did nothing would be caught
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(scanned, eager[0]) and torch.equal(C, eager[1]) and torch.equal(D, eager[2])
        assert np.array_equal(scanned.cpu().numpy(), oracle.scan_cpu(oracle.add_m(xs, 7)))
        want = oracle.np_sgemm_f64(1.0, a, b, 1.0, oracle.np_sgemm_f64(1.5, a, b, 0.5, c).astype(np.float32))
        tol = 2 * oracle.sgemm_tolerance(K, a, b) + 2.0**-20
        assert np.max(np.abs(C.cpu().numpy() - want)) <= tol
        ref = oracle.gemm_bf16_f64(p16, q16)
        assert np.max(np.abs(D.cpu().numpy() - ref)) <= 1e-3 * np.abs(ref).max()
    prism.scan_status(ws)
