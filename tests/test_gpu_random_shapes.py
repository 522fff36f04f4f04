"""Seeded random shapes and alignments through the two MFMA GEMMs, every element against an fp64 product.

The hand-picked shapes of test_gpu_sgemm.py and test_gpu_gemm_bf16.py sit on the boundaries the launchers
know about; these draws land between them: any M, N, K from 1 up (K up to 4000: beyond about 8000 the rounding of
a single fp32 sum chain, rocBLAS's included, reaches the sqrt(K) bound used here), operands that start at any
element of their buffers (so rows are 4 B, 8 B or 16 B aligned for fp32 and 2 B to 16 B aligned for bf16), beta
zero or not, and where the workspace form of the SGEMM would cut K, that form as well.
The operands sit between NaNs and the output between guard values, so a read outside a matrix or a store
outside the output shows. The fp64 product is formed on the device (torch), which keeps the test short; the
bounds are the ones of the hand-picked tests (1e-5 sqrt(K) max|A| max|B| for fp32, 1e-3 of the largest
|element| for bf16).
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _draw_shapes(seed, count, big):
    rng = np.random.default_rng(seed)
    out = []
    for i in range(count):
        kind = i % 6
        if kind == 0:      # small: one-wave tiles, K from 1 up
            M, N, K = rng.integers(1, 200), rng.integers(1, 200), rng.integers(1, 100)
        elif kind == 1:    # a few hundred: rings, one-wave tiles with K split off
            M, N, K = rng.integers(100, 900), rng.integers(100, 900), rng.integers(4, 600)
        elif kind == 2:    # one long side
            M, N, K = rng.integers(1, 64), rng.integers(500, 3000), rng.integers(8, 300)
            if rng.integers(0, 2):
                M, N = N, M
        elif kind == 3:    # mid sizes: workgroup tiles, partial rounds
            M, N, K = rng.integers(1500, big), rng.integers(1500, big), rng.integers(16, 200)
        elif kind == 4:    # few tiles and a long K: K cut inside the workgroup, long rings
            M, N, K = rng.integers(1, 300), rng.integers(1, 1100), rng.integers(1000, 4000)
        else:              # whole multiples of the tiles: the forms without range checks, when the starts allow
            M, N, K = 64 * rng.integers(1, 12), 256 * rng.integers(1, 10), 16 * rng.integers(8, 250)
        starts = [int(rng.integers(0, 8)), int(rng.integers(0, 8)), int(rng.integers(0, 4))]
        if kind == 5 and rng.integers(0, 2):
            starts = [0, 0, 0]
        out.append((int(M), int(N), int(K), *starts))
    return out


def _fenced(values: torch.Tensor, start: int, fill) -> torch.Tensor:
    """`values` as a view that starts at element `start` of a buffer otherwise filled with `fill`."""
    buf = torch.full((values.numel() + 64,), fill, dtype=values.dtype, device=DEV)
    view = buf[start:start + values.numel()].view(values.shape)
    view.copy_(values)
    return view


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_sgemm_kernel_5_random_shapes(prism, seed):
    g = torch.Generator(device=DEV)
    g.manual_seed(seed)
    for (M, N, K, sa, sb, sc) in _draw_shapes(seed, 72, 4700):
        A = torch.rand((M, K), device=DEV, generator=g) * 2 - 1
        B = torch.rand((K, N), device=DEV, generator=g) * 2 - 1
        C0 = torch.rand((M, N), device=DEV, generator=g) * 2 - 1
        beta = 0.5 if (M + N + K) % 2 else 0.0
        a, b = _fenced(A, sa % 4, float("nan")), _fenced(B, sb % 4, float("nan"))
        cbuf = torch.full((M * N + 64,), 777.0, device=DEV)
        c = cbuf[8 + sc:8 + sc + M * N].view(M, N)
        c.copy_(C0)
        print(f"sgemm M={M} N={N} K={K} starts {sa % 4} {sb % 4} {8 + sc} beta={beta}", flush=True)
        prism.sgemm(M, N, K, 1.25, a, b, beta, c, variant=5)
        torch.cuda.synchronize()
        assert bool((cbuf[:8 + sc] == 777.0).all()) and bool((cbuf[8 + sc + M * N:] == 777.0).all())
        want = 1.25 * (A.double() @ B.double()) + beta * C0.double()
        err = float((c.double() - want).abs().max())
        assert err <= 1e-5 * np.sqrt(K) + abs(beta) * 2**-22, f"{M}x{N}x{K}: max error {err:.3e}"
        ws_bytes = prism.sgemm_workspace_size(M, N, K)
        if ws_bytes:     # the same product through the entry point that may cut K across workgroups
            ws = torch.full((ws_bytes // 4,), float("nan"), device=DEV)
            c.copy_(C0)
            prism.sgemm(M, N, K, 1.25, a, b, beta, c, variant=5, workspace=ws)
            torch.cuda.synchronize()
            assert bool((cbuf[:8 + sc] == 777.0).all()) and bool((cbuf[8 + sc + M * N:] == 777.0).all())
            err = float((c.double() - want).abs().max())
            assert err <= 1e-5 * np.sqrt(K) + abs(beta) * 2**-22, f"{M}x{N}x{K} with a workspace: max error {err:.3e}"


@pytest.mark.parametrize("seed", [11, 12])
def test_sgemm_random_shapes_with_more_tiles_than_cus(prism, seed):
    """Draws the ones above do not reach: more 256 x 256 tiles than CUs, K on both sides of 2048 (up to there the whole
    rounds run as 128 x 256 halves; from there on the workspace form shares the last round's K loops between all
    workgroups (ragged M and any start; N, K multiples of 4 or not:
    the shared form needs 16 B-aligned rows and is asked for only then), and a thin strip of columns beyond a whole
    number of tiles. Both entry points, every element, guard values around C, a workspace full of NaN. (The same
    draws over 28 000 more seeds were run once.)"""
    rng = np.random.default_rng(seed)
    g = torch.Generator(device=DEV)
    g.manual_seed(seed)
    taken = 0
    for i in range(9):
        kind = i % 3
        if kind == 0:
            M, N, K = int(rng.integers(4100, 6200)), int(rng.integers(4100, 6200)), int(rng.integers(1500, 2600))
        elif kind == 1:
            M, N, K = int(rng.integers(4100, 6200)), 4 * int(rng.integers(1025, 1550)), 4 * int(rng.integers(512, 650))
        else:
            M, N, K = int(rng.integers(64, 3000)), 256 * int(rng.integers(1, 12)) + int(rng.integers(1, 9)), int(rng.integers(16, 1200))
        sa, sb, sc = (int(rng.integers(0, 4)) for _ in range(3))
        if kind == 1 and i % 2:
            sa = sb = sc = 0
        A = torch.rand((M, K), device=DEV, generator=g) * 2 - 1
        B = torch.rand((K, N), device=DEV, generator=g) * 2 - 1
        C0 = torch.rand((M, N), device=DEV, generator=g) * 2 - 1
        beta = 0.5 if i % 2 else 0.0
        a, b = _fenced(A, sa, float("nan")), _fenced(B, sb, float("nan"))
        cbuf = torch.full((M * N + 64,), 777.0, device=DEV)
        c = cbuf[8 + sc:8 + sc + M * N].view(M, N)
        want = 1.25 * (A.double() @ B.double()) + beta * C0.double()
        ws_bytes = prism.sgemm_workspace_size(M, N, K)
        ws = torch.full((max(ws_bytes, 4) // 4,), float("nan"), device=DEV)
        for use_ws in (False, True):
            c.copy_(C0)
            print(f"sgemm M={M} N={N} K={K} starts {sa} {sb} {8 + sc} beta={beta} workspace={use_ws and ws_bytes}", flush=True)
            prism.sgemm(M, N, K, 1.25, a, b, beta, c, variant=5, workspace=ws if use_ws else None)
            torch.cuda.synchronize()
            assert bool((cbuf[:8 + sc] == 777.0).all()) and bool((cbuf[8 + sc + M * N:] == 777.0).all())
            err = float((c.double() - want).abs().max())
            assert err <= 1e-5 * np.sqrt(K) + abs(beta) * 2**-22, f"{M}x{N}x{K} workspace={use_ws}: max error {err:.3e}"
        if sa == 0 and sb == 0 and (8 + sc) % 4 == 0:
            taken += prism.sgemm_workspace_plan(M, N, K, ws_bytes)[0] > 0
    assert taken >= 1   # at least one draw went through the shared form


@pytest.mark.parametrize("seed", [4, 5, 6])
def test_gemm_bf16_random_shapes(prism, seed):
    g = torch.Generator(device=DEV)
    g.manual_seed(seed)
    nan16 = torch.tensor(float("nan"), dtype=torch.bfloat16)
    for (M, N, K, sa, sb, sc) in _draw_shapes(seed, 72, 4700):
        A = torch.randn((M, K), device=DEV, generator=g).to(torch.bfloat16)
        B = torch.randn((N, K), device=DEV, generator=g).to(torch.bfloat16)
        a, b = _fenced(A, sa, nan16.item()), _fenced(B, sb, nan16.item())
        dbuf = torch.full((M * N + 64,), 777.0, device=DEV)
        d = dbuf[8 + sc:8 + sc + M * N].view(M, N)
        print(f"gemm_bf16 M={M} N={N} K={K} starts {sa} {sb} {8 + sc}", flush=True)
        prism.gemm_bf16(a, b, d)
        torch.cuda.synchronize()
        assert bool((dbuf[:8 + sc] == 777.0).all()) and bool((dbuf[8 + sc + M * N:] == 777.0).all())
        want = A.double() @ B.double().t()
        err = float((d.double() - want).abs().max())
        assert err <= 1e-3 * float(want.abs().max()), f"{M}x{N}x{K}: max error {err:.3e}"
        if K % 2 == 0:   # the bf16 column-major form on every other draw
            cbuf = torch.full((N * M + 64,), -7.0, dtype=torch.bfloat16, device=DEV)
            cc = cbuf[8 + sc:8 + sc + N * M]
            prism.runmyh100(M, N, K, a, b, cc)
            torch.cuda.synchronize()
            assert bool((cbuf[:8 + sc] == -7.0).all()) and bool((cbuf[8 + sc + N * M:] == -7.0).all())
            got = cc.view(N, M).t().double()
            assert bool(((got - want).abs() <= 2.0**-8 * want.abs() + 1e-3 * float(want.abs().max())).all())


@pytest.mark.parametrize("seed", [7, 8])
def test_scans_random_lengths_and_alignments(prism, seed):
    """Random lengths (1 to 2^25, both tile shapes and their edges), first elements at any index (4 B to 16 B
    aligned), in place or not, one workspace for all calls and kinds; against torch's scans on the device,
    bit for bit."""
    rng = np.random.default_rng(seed)
    g = torch.Generator(device=DEV)
    g.manual_seed(seed)
    ws = prism.new_scan_workspace(1 << 25)
    for i in range(40):
        n = int(rng.integers(1, 1 << int(rng.integers(1, 26))))
        start, kind, in_place = int(rng.integers(0, 4)), int(rng.integers(0, 4)), bool(rng.integers(0, 2))
        buf = torch.randint(-1000, 1001, (n + 8,), dtype=torch.int32, device=DEV, generator=g)
        if kind == 0:
            buf[start] += 2**31 - 1000      # the sums wrap around
        x = buf[start:start + n]
        keep = x.clone()
        out = x if in_place else torch.full((n + 8,), 12345, dtype=torch.int32, device=DEV)[4 - start:4 - start + n]
        print(f"scan n={n} start={start} kind={kind} in_place={in_place}", flush=True)
        if kind in (0, 1):
            got = prism.scan(x, out=out, workspace=ws)
            want = torch.cumsum(keep, 0, dtype=torch.int32)
        elif kind == 2:
            got = prism.scan(x, out=out, workspace=ws, exclusive=True)
            want = torch.cumsum(keep, 0, dtype=torch.int32) - keep
        else:
            got = prism.scan(x, out=out, workspace=ws, op="max")
            want = torch.cummax(keep, 0).values
        assert torch.equal(got, want), f"n={n} start={start} kind={kind}"
        if not in_place:
            assert torch.equal(x, keep)
        if i % 4 == 0:   # the same call with look-backs that never wait: every silent predecessor is helped
            if in_place:
                x.copy_(keep)
            kw = {"exclusive": True} if kind == 2 else {"op": "max"} if kind == 3 else {}
            assert torch.equal(prism.scan(x, out=out, workspace=ws, spin_limit=0, **kw), want), f"n={n} start={start} kind={kind} helping"
