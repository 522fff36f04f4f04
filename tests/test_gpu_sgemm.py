"""GPU parity tests for the fp32 SGEMM progression, through the C ABI.

Kernels 1, 2, 3, 4, 6 compute each element as a serial chain of fused
multiply-adds over increasing k, so they must equal the fmaf oracle BIT FOR BIT.
Kernel 5 (MFMA) is checked against the fp64 oracle with the tolerance
max|err| <= 1e-5 * sqrt(K) * max|A| * max|B| (plus the rounding of the beta*C term).
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
EXACT = (1, 2, 3, 4, 6)
ALL = (1, 2, 3, 4, 5, 6)


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def run(prism, variant, alpha, A, B, beta, Cm):
    M, K = A.shape
    N = B.shape[1]
    c = dev(Cm).clone()
    prism.sgemm(M, N, K, alpha, dev(A), dev(B), beta, c, variant=variant)
    return host(c)


def tol(oracle, K, A, B, beta, Cm):
    extra = abs(beta) * float(np.abs(Cm).max(initial=0.0)) * 2**-22 if beta != 0 else 0.0
    return oracle.sgemm_tolerance(K, A, B) + extra


SMALL = [(1, 1, 1), (16, 16, 16), (33, 47, 29), (127, 129, 17), (64, 64, 64), (128, 128, 128),
         (130, 70, 33), (256, 128, 64), (64, 200, 8), (200, 64, 250), (129, 257, 100)]


@pytest.mark.parametrize("shape", SMALL)
def test_exact_kernels_match_fma_oracle_bitwise(prism, oracle, shape):
    M, N, K = shape
    A, B, Cm = oracle.gen_sgemm(M, N, K, seed=M + N + K)
    want = oracle.sgemm_fma(0.5, A, B, 3.0, Cm)
    for v in EXACT:
        got = run(prism, v, 0.5, A, B, 3.0, Cm)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), f"kernel {v} shape {shape}"


@pytest.mark.parametrize("shape", SMALL)
def test_wave_tile_kernel_within_tolerance(prism, oracle, shape):
    M, N, K = shape
    A, B, Cm = oracle.gen_sgemm(M, N, K, seed=M + N + K)
    want = oracle.sgemm_f64(1.0, A, B, 0.5, Cm)
    got = run(prism, 5, 1.0, A, B, 0.5, Cm)
    assert np.max(np.abs(got - want)) <= tol(oracle, K, A, B, 0.5, Cm)
    # variant 0 is the alias of the best kernel
    assert np.array_equal(run(prism, 0, 1.0, A, B, 0.5, Cm), got)


def test_fixture(prism, golden, oracle):
    a, b = (float(v) for v in golden["sgemm_alpha_beta"])
    A, B, Cm = golden["sgemm_A"], golden["sgemm_B"], golden["sgemm_C"]
    for v in EXACT:
        assert np.array_equal(run(prism, v, a, A, B, b, Cm), golden["sgemm_out_fma"])
    got = run(prism, 5, a, A, B, b, Cm)
    assert np.max(np.abs(got - golden["sgemm_out_f64"])) <= tol(oracle, A.shape[1], A, B, b, Cm)


def test_reference_harness_configuration(prism, oracle):
    """The reference's own correctness run: 1024^3, alpha 0.5, beta 3.0, entries +-(k + 0.01 j),
    k, j in 0..4, every kernel within 0.01 of the oracle (evals/4090_sgemm/main.cu:48,84-147,
    runner.cu:54-65,105-117), through run_my_kernel."""
    n = 1024
    rng = np.random.default_rng(1)

    def randomize(shape):
        v = rng.integers(0, 5, shape).astype(np.float32) + np.float32(0.01) * rng.integers(0, 5, shape).astype(np.float32)
        return np.where(rng.integers(0, 2, shape) == 0, v, -v).astype(np.float32)

    A, B, Cm = randomize((n, n)), randomize((n, n)), randomize((n, n))
    want = oracle.np_sgemm_f64(0.5, A, B, 3.0, Cm)
    for k in (1, 2, 3, 4, 5):
        c = dev(Cm).clone()
        prism.run_my_kernel(k, n, n, n, 0.5, dev(A), dev(B), 3.0, c)
        got = host(c)
        assert np.max(np.abs(got - want)) <= 0.01, f"kernel {k}"
        assert np.max(np.abs(got - want)) <= tol(oracle, n, A, B, 3.0, Cm), f"kernel {k}"
    with pytest.raises(ValueError):
        prism.run_my_kernel(6, n, n, n, 0.5, dev(A), dev(B), 3.0, dev(Cm))


def test_special_cases_all_kernels(prism, oracle):
    M, N, K = 96, 160, 72
    A, B, Cm = oracle.gen_sgemm(M, N, K, seed=3)
    poison = np.full((M, N), np.nan, dtype=np.float32)
    eye = np.eye(K, dtype=np.float32)
    for v in ALL:
        # beta == 0 never reads C
        got = run(prism, v, 1.0, A, B, 0.0, poison)
        assert np.isfinite(got).all(), f"kernel {v} read C with beta == 0"
        assert np.max(np.abs(got - oracle.sgemm_f64(1.0, A, B, 0.0))) <= oracle.sgemm_tolerance(K, A, B)
        # alpha == 0: C = beta * C exactly
        assert np.array_equal(run(prism, v, 0.0, A, B, 0.5, Cm), np.float32(0.5) * Cm), f"kernel {v}"
        # B = I: C = A exactly (0 and 1 products are exact in every summation order)
        assert np.array_equal(run(prism, v, 1.0, A, eye, 0.0, np.zeros((M, K), np.float32)), A), f"kernel {v}"
        # K == 1 outer product, K == 0 scaling
        a1, b1 = A[:, :1].copy(), B[:1, :].copy()
        assert np.array_equal(run(prism, v, 1.0, a1, b1, 0.0, poison), a1 * b1), f"kernel {v}"
        a0, b0 = np.zeros((M, 0), np.float32), np.zeros((0, N), np.float32)
        assert np.array_equal(run(prism, v, 1.0, a0, b0, 2.0, Cm), 2.0 * Cm), f"kernel {v}"


def test_does_not_write_outside_c(prism, oracle):
    M, N, K = 70, 45, 33
    A, B, Cm = oracle.gen_sgemm(M, N, K, seed=5)
    for v in ALL:
        buf = torch.full((M * N + 512,), 777.0, dtype=torch.float32, device=DEV)
        c = buf[256:256 + M * N]
        c.copy_(dev(Cm).reshape(-1))
        prism.sgemm(M, N, K, 1.0, dev(A), dev(B), 0.5, c, variant=v)
        out = host(buf)
        assert np.all(out[:256] == 777.0) and np.all(out[256 + M * N:] == 777.0), f"kernel {v}"


@pytest.mark.parametrize("n", [1024, 2048])
def test_baseline_square_all_kernels(prism, oracle, n):
    A, B, Cm = oracle.gen_sgemm(n, n, n, seed=0)
    want = oracle.np_sgemm_f64(1.0, A, B, 0.5, Cm)
    t = tol(oracle, n, A, B, 0.5, Cm)
    first = None
    for v in ALL:
        got = run(prism, v, 1.0, A, B, 0.5, Cm)
        assert np.max(np.abs(got - want)) <= t, f"kernel {v} n {n}"
        if v in EXACT:
            first = got if first is None else first
            assert np.array_equal(got, first), f"kernel {v} differs from kernel 1 bitwise"


@pytest.mark.parametrize("shape", [(4096, 4096, 128), (128, 4096, 4096), (8191, 4097, 1023)])
def test_baseline_tail_shapes(prism, oracle, shape):
    M, N, K = shape
    A, B, _ = oracle.gen_sgemm(M, N, K, seed=1)
    want = oracle.np_sgemm_f64(1.0, A, B, 0.0)
    poison = np.full((M, N), np.nan, dtype=np.float32)
    t = oracle.sgemm_tolerance(K, A, B)
    for v in (4, 5):
        got = run(prism, v, 1.0, A, B, 0.0, poison)
        assert np.max(np.abs(got - want)) <= t, f"kernel {v} shape {shape}"


@pytest.mark.parametrize("shape", [(4096, 4096, 16), (4096, 4096, 32), (4096, 4096, 48), (4096, 4096, 80),
                                   (2048, 8192, 96), (8192, 2048, 64)])
def test_wave_tile_whole_tile_path(prism, oracle, shape):
    """Shapes made of whole 256 x 256 tiles, enough for three quarters of the CUs, take kernel 5's direct-to-LDS path; K covers
    one, an even and an odd number of K tiles. Every element is checked, with and without reading C,
    and against the general path (same data at a 4-byte offset, which the whole-tile path rejects)."""
    M, N, K = shape
    A, B, Cm = oracle.gen_sgemm(M, N, K, seed=K)
    t = tol(oracle, K, A, B, -0.5, Cm)
    got = run(prism, 5, 1.5, A, B, -0.5, Cm)
    assert np.max(np.abs(got - oracle.np_sgemm_f64(1.5, A, B, -0.5, Cm))) <= t
    poison = np.full((M, N), np.nan, dtype=np.float32)
    got0 = run(prism, 5, 1.0, A, B, 0.0, poison)
    assert np.max(np.abs(got0 - oracle.np_sgemm_f64(1.0, A, B, 0.0))) <= oracle.sgemm_tolerance(K, A, B)
    buf = torch.full((M * N + 8,), 777.0, dtype=torch.float32, device=DEV)
    c = buf[1:1 + M * N]
    c.copy_(dev(Cm).reshape(-1))
    prism.sgemm(M, N, K, 1.5, dev(A), dev(B), -0.5, c, variant=5)
    out = host(buf)
    assert out[0] == 777.0 and np.all(out[1 + M * N:] == 777.0)
    assert np.max(np.abs(out[1:1 + M * N].reshape(M, N) - got)) <= 2 * t


@pytest.mark.parametrize("shape", [(512, 512, 64), (1024, 1024, 80), (1024, 1024, 96), (1024, 1024, 112), (1024, 512, 256),
                                   (2048, 2048, 128), (128, 4096, 256), (64, 64, 2048), (96, 160, 64),
                                   (128, 2048, 512), (128, 2048, 544), (64, 1024, 1024), (128, 128, 4096), (512, 512, 1088),
                                   (64, 4096, 2048), (32, 32, 1024), (32, 64, 1216)])
def test_wave_tile_one_wave_per_tile_path(prism, oracle, shape):
    """Problems with at most one 64 x 64 tile per SIMD take kernel 5's one-wave-per-tile path (32 x 32
    tiles below that, 64 x 64 at exactly that); K covers every residue of the 4-stage ring. The second row
    of shapes has at most a quarter as many 32 x 32 tiles as there are SIMDs and a long K: two or four waves share a tile, each with a
    part of K (every residue of the ring again), and add up in LDS. Every element is checked, with and
    without reading C, and a second run gives the same bits."""
    M, N, K = shape
    A, B, Cm = oracle.gen_sgemm(M, N, K, seed=K + N)
    got = run(prism, 5, -0.75, A, B, 2.0, Cm)
    assert np.max(np.abs(got - oracle.np_sgemm_f64(-0.75, A, B, 2.0, Cm))) <= tol(oracle, K, A, B, 2.0, Cm)
    poison = np.full((M, N), np.nan, dtype=np.float32)
    got0 = run(prism, 5, 1.0, A, B, 0.0, poison)
    assert np.max(np.abs(got0 - oracle.np_sgemm_f64(1.0, A, B, 0.0))) <= oracle.sgemm_tolerance(K, A, B)
    assert np.array_equal(run(prism, 5, -0.75, A, B, 2.0, Cm), got)


@pytest.mark.parametrize("shape", [(4352, 4352, 64), (4096, 5120, 80), (5120, 5120, 80), (5120, 5120, 48), (4608, 4608, 64),
                                   (4096, 4352, 96), (4864, 4864, 64), (4736, 4740, 68)])
def test_wave_tile_leftover_round(prism, oracle, shape):
    """Whole 256 x 256 tiles that do not fill whole rounds of the 256 CUs: the last, partial round is cut
    into smaller tiles by a second launch: 64 x 256 slices of the same kernel when that gives every CU one
    (289 tiles: 33 left over; 320: 64 left over) or three (400: 144 left over), else one-wave tiles (324: 68 left
    over as 64 x 64 tiles; 272: 16 left over as 32 x 32), and 128 x 256 halves for 80 to 128 tiles left over (361
    tiles: 105 left over, whole and ragged). With K below 64 (fourth shape) the big kernel takes every tile. Every
    element is checked."""
    M, N, K = shape
    A, B, Cm = oracle.gen_sgemm(M, N, K, seed=M + K)
    got = run(prism, 5, 1.25, A, B, 0.5, Cm)
    assert np.max(np.abs(got - oracle.np_sgemm_f64(1.25, A, B, 0.5, Cm))) <= tol(oracle, K, A, B, 0.5, Cm)


@pytest.mark.parametrize("shape", [(128, 4096, 4096), (64, 2048, 8192), (256, 256, 16384), (192, 768, 8192), (64, 4096, 4096)])
def test_wave_tile_k_split_with_workspace(prism, oracle, shape):
    """Skinny products through prism_sgemm_ws: the K ranges of the few 64 x 256 tiles are shared between all
    CUs, every workgroup writes its partial products into the workspace and a second kernel adds a tile's parts
    in the order of k. Every element against fp64, with and without reading C (C full of NaN when it is not
    read), the same bits on a second run, nothing written beyond the bytes prism_sgemm_workspace_bytes names,
    and with a workspace one byte short the call is the unshared one, bit for bit."""
    M, N, K = shape
    need = prism.sgemm_workspace_size(M, N, K)
    groups, shared = prism.sgemm_workspace_plan(M, N, K, need)
    assert shared == (M // 64) * (N // 256) and 2 * shared <= groups <= prism.device_info()["cu_count"]
    assert need == 2 * groups * 64 * 256 * 4 and prism.sgemm_workspace_plan(M, N, K, need - 1) == (0, 0)
    A, B, Cm = oracle.gen_sgemm(M, N, K, seed=M + N + K)
    a, b = dev(A), dev(B)
    wsbuf = torch.full((need + 512,), 0x5A, dtype=torch.uint8, device=DEV)
    ws = wsbuf[256:256 + need]
    outs = []
    for beta, c0 in ((0.5, Cm), (0.0, np.full((M, N), np.nan, dtype=np.float32))):
        c = dev(c0).clone()
        prism.sgemm(M, N, K, 1.25, a, b, beta, c, variant=5, workspace=ws)
        got = host(c)
        assert np.max(np.abs(got - oracle.np_sgemm_f64(1.25, A, B, beta, Cm))) <= tol(oracle, K, A, B, beta, Cm)
        c2 = dev(c0).clone()
        prism.sgemm(M, N, K, 1.25, a, b, beta, c2, variant=5, workspace=ws)
        assert np.array_equal(host(c2), got)
        outs.append(got)
    guard = host(wsbuf)
    assert np.all(guard[:256] == 0x5A) and np.all(guard[256 + need:] == 0x5A)
    short = torch.empty(need - 1, dtype=torch.uint8, device=DEV)
    c3, c4 = dev(Cm).clone(), dev(Cm).clone()
    prism.sgemm(M, N, K, 1.25, a, b, 0.5, c3, variant=5, workspace=short)
    prism.sgemm(M, N, K, 1.25, a, b, 0.5, c4, variant=5)
    assert np.array_equal(host(c3), host(c4))
    assert np.max(np.abs(host(c3) - outs[0])) <= 2 * tol(oracle, K, A, B, 0.5, Cm)


@pytest.mark.parametrize("shape", [(4352, 4352, 2048), (5120, 5120, 2080), (5000, 5000, 2052), (4608, 4864, 3072), (4228, 4612, 2060), (4100, 5376, 2052)])
def test_wave_tile_last_round_shared_with_workspace(prism, oracle, shape):
    """256 x 256 tiles that are not a whole number of rounds of the CUs, through prism_sgemm_ws: the whole rounds
    run one tile per workgroup, the K ranges of the tiles of the last round (33, 144, 144, 86, 67 and 80 beside a strip of four rows here) are
    shared between all CUs, and a second kernel adds a tile's partial products (K of 2048 and up: below that the
    entry point leaves the product to prism_sgemm, see test_short_k_is_not_shared). Whole tiles and ragged M, N, K
    (rows 16 B aligned). Every element against an fp64 product formed on the
    device, with and without reading C (NaN in C when it is not read), the same bits on a second run, nothing
    written outside the workspace, and the plan query says that the shared form is the one that ran."""
    import fp64_referee
    M, N, K = shape
    cus = prism.device_info()["cu_count"]
    tiles = (M // 256 if 0 < M % 256 <= 8 else -(-M // 256)) * -(-N // 256)   # up to 8 rows beyond whole tiles go to the strip kernel
    need = prism.sgemm_workspace_size(M, N, K)
    assert need == 2 * cus * 256 * 256 * 4
    assert prism.sgemm_workspace_plan(M, N, K, need) == (cus, tiles % cus)
    A, B, C0 = _device_inputs(M, N, K)
    wsbuf = torch.full((need + 512,), 0x5A, dtype=torch.uint8, device=DEV)
    ws = wsbuf[256:256 + need]
    for beta in (0.5, 0.0):
        c = C0.clone() if beta else torch.full((M, N), float("nan"), device=DEV)
        print(f"prism_sgemm_ws {M}x{N}x{K} beta={beta}", flush=True)
        prism.sgemm(M, N, K, 1.25, A, B, beta, c, variant=5, workspace=ws)
        err = fp64_referee.sgemm_max_err_fp64(1.25, A, B, beta, C0, c)
        assert err <= 1.25 * _bound(K, beta), f"{M}x{N}x{K} beta={beta}: max error {err:.3e}"
        c2 = C0.clone() if beta else torch.full((M, N), float("nan"), device=DEV)
        prism.sgemm(M, N, K, 1.25, A, B, beta, c2, variant=5, workspace=ws)
        assert torch.equal(c, c2)
    assert bool((wsbuf[:256] == 0x5A).all()) and bool((wsbuf[256 + need:] == 0x5A).all())


def test_short_k_is_not_shared(prism):
    """With a short K a tile holds too little work to pay for partial products: no workspace is asked for, and
    the workspace entry point gives the bits of the plain one."""
    for (M, N, K) in ((5120, 5120, 512), (4352, 4352, 1024), (4100, 4612, 300)):
        assert prism.sgemm_workspace_size(M, N, K) == 0 and prism.sgemm_workspace_plan(M, N, K, 1 << 30) == (0, 0)
    M, N, K = 4352, 4352, 1024
    A, B, C0 = _device_inputs(M, N, K)
    ws = torch.empty(1 << 20, device=DEV)
    c1, c2 = C0.clone(), C0.clone()
    prism.sgemm(M, N, K, 1.25, A, B, 0.5, c1, variant=5, workspace=ws)
    prism.sgemm(M, N, K, 1.25, A, B, 0.5, c2, variant=5)
    assert torch.equal(c1, c2)


@pytest.mark.parametrize("shape", [(4096, 4096, 128), (8192, 4096, 256), (4100, 4612, 300), (8190, 4098, 1000), (4097, 4097, 1025), (5120, 5120, 512), (4096, 8192, 2048)])
def test_wave_tile_short_k_runs_as_halves(prism, oracle, shape):
    """K up to 2048 on problems with at least as many 256 x 256 tiles as CUs: the tiles of the whole rounds run as
    128 x 256 halves, two workgroups to a CU (whole tiles, ragged edges, rows that are only 4 B aligned, a partial
    last round beside them). Every element against fp64, with and without reading C, guard values around C."""
    import fp64_referee
    M, N, K = shape
    A, B, C0 = _device_inputs(M, N, K)
    for beta in (0.5, 0.0):
        cbuf = torch.full((M * N + 128,), 777.0, device=DEV)
        c = cbuf[64:64 + M * N].view(M, N)
        c.copy_(C0 if beta else torch.full((M, N), float("nan"), device=DEV))
        print(f"prism_sgemm {M}x{N}x{K} beta={beta}", flush=True)
        prism.sgemm(M, N, K, 0.75, A, B, beta, c, variant=5)
        err = fp64_referee.sgemm_max_err_fp64(0.75, A, B, beta, C0, c)
        assert err <= _bound(K, beta), f"{M}x{N}x{K} beta={beta}: max error {err:.3e}"
        assert bool((cbuf[:64] == 777.0).all()) and bool((cbuf[64 + M * N:] == 777.0).all())


@pytest.mark.parametrize("shape", [(4097, 4097, 1025), (4100, 4096, 512), (8193, 4100, 300), (4104, 4104, 2100), (4098, 6000, 17), (4097, 4096, 4096)])
def test_wave_tile_thin_strip_of_rows(prism, oracle, shape):
    """M a few rows (1 to 8) beyond a whole number of 256-row tiles: the rows before run as ever, a strip kernel
    takes the rest (with a thin strip of columns at the same time, ragged N and K, K shorter than its sixteen
    wavefronts' shares and longer than one trip of their loops). Every element against fp64; C poisoned with
    NaN when it is not read; guard values around C; operands that start at an odd element."""
    import fp64_referee
    M, N, K = shape
    A0, B0, C0 = _device_inputs(M, N, K)
    for beta, shift in ((0.5, 0), (0.0, 1)):
        abuf = torch.full((M * K + 8,), float("nan"), device=DEV)
        bbuf = torch.full((K * N + 8,), float("nan"), device=DEV)
        A, B = abuf[shift:shift + M * K].view(M, K), bbuf[shift:shift + K * N].view(K, N)
        A.copy_(A0)
        B.copy_(B0)
        cbuf = torch.full((M * N + 128,), 777.0, device=DEV)
        c = cbuf[64 + shift:64 + shift + M * N].view(M, N)
        c.copy_(C0 if beta else torch.full((M, N), float("nan"), device=DEV))
        print(f"prism_sgemm {M}x{N}x{K} beta={beta} operands start at element {shift}", flush=True)
        prism.sgemm(M, N, K, 0.75, A, B, beta, c, variant=5)
        err = fp64_referee.sgemm_max_err_fp64(0.75, A0, B0, beta, C0, c)
        assert err <= _bound(K, beta), f"{M}x{N}x{K} beta={beta}: max error {err:.3e}"
        assert bool((cbuf[:64 + shift] == 777.0).all()) and bool((cbuf[64 + shift + M * N:] == 777.0).all())


@pytest.mark.parametrize("shape", [(4096, 3073, 100), (4000, 3080, 67), (4096, 3076, 64), (8191, 4097, 1023), (4096, 3329, 4), (3000, 4099, 2100)])
def test_wave_tile_thin_strip_of_columns(prism, oracle, shape):
    """N a few columns (1 to 8) beyond a whole number of 256-column tiles: the big tiles take the whole tile
    columns, a strip kernel the rest (rows 4 B or 16 B aligned, whole and ragged M and K, K longer than the
    strip kernel's LDS chunk). Every element against fp64; C poisoned with NaN when it is not read; guard
    values around C."""
    import fp64_referee
    M, N, K = shape
    A, B, C0 = _device_inputs(M, N, K)
    for beta in (0.5, 0.0):
        cbuf = torch.full((M * N + 128,), 777.0, device=DEV)
        c = cbuf[64:64 + M * N].view(M, N)
        c.copy_(C0 if beta else torch.full((M, N), float("nan"), device=DEV))
        print(f"prism_sgemm {M}x{N}x{K} beta={beta}", flush=True)
        prism.sgemm(M, N, K, 0.75, A, B, beta, c, variant=5)
        err = fp64_referee.sgemm_max_err_fp64(0.75, A, B, beta, C0, c)
        assert err <= _bound(K, beta), f"{M}x{N}x{K} beta={beta}: max error {err:.3e}"
        assert bool((cbuf[:64] == 777.0).all()) and bool((cbuf[64 + M * N:] == 777.0).all())


def test_workspace_form_leaves_other_shapes_and_kernels_alone(prism, oracle):
    """Shapes the split is not for, and the kernels other than 5, run as in prism_sgemm: same bits with and
    without a workspace."""
    ws = torch.empty(64 << 20, dtype=torch.uint8, device=DEV)
    for (M, N, K, variant) in ((1024, 1024, 1024, 5), (128, 4096, 1000, 5), (100, 4096, 4096, 5), (128, 4096, 4096, 4), (128, 4096, 4096, 1)):
        assert variant != 5 or prism.sgemm_workspace_size(M, N, K) == 0
        A, B, Cm = oracle.gen_sgemm(M, N, K, seed=K)
        c1, c2 = dev(Cm).clone(), dev(Cm).clone()
        prism.sgemm(M, N, K, 1.0, dev(A), dev(B), 0.5, c1, variant=variant, workspace=ws)
        prism.sgemm(M, N, K, 1.0, dev(A), dev(B), 0.5, c2, variant=variant)
        assert np.array_equal(host(c1), host(c2))


def nan_fenced(a: np.ndarray, start: int = 1024) -> torch.Tensor:
    """The matrix as a view into a device buffer whose other elements are NaN; `start` is its first
    element's index (a multiple of 4 keeps it 16 B aligned)."""
    buf = torch.full((a.size + 2048,), float("nan"), dtype=torch.float32, device=DEV)
    buf[start:start + a.size] = torch.from_numpy(np.ascontiguousarray(a).ravel()).to(DEV)
    return buf[start:start + a.size].view(a.shape)


@pytest.mark.parametrize("shape", [(1000, 1001, 999), (515, 777, 130), (128, 128, 16), (1, 1500, 7), (1500, 2, 3), (640, 640, 64)])
def test_wave_tile_any_shape_between_nans(prism, oracle, shape):
    """The general kernel 5 path: any M, N, K, operands only 4 B aligned (their first element sits at an
    odd index). Its edge tiles are filled by range-checked 16 B buffer loads plus masks for what lies past
    a row's end; A and B sit between NaNs, so a read outside a matrix or a missing mask poisons the output."""
    M, N, K = shape
    A, B, Cm = oracle.gen_sgemm(M, N, K, seed=M + 5 * K)
    for start in (1024, 1021):
        buf = torch.full((M * N + 512,), 777.0, dtype=torch.float32, device=DEV)
        c = buf[255:255 + M * N].view(M, N)
        c.copy_(dev(Cm))
        prism.sgemm(M, N, K, 1.25, nan_fenced(A, start), nan_fenced(B, start), 0.5, c, variant=5)
        out = host(buf)
        assert np.all(out[:255] == 777.0) and np.all(out[255 + M * N:] == 777.0)
        got = out[255:255 + M * N].reshape(M, N)
        assert np.max(np.abs(got - oracle.np_sgemm_f64(1.25, A, B, 0.5, Cm))) <= tol(oracle, K, A, B, 0.5, Cm)


@pytest.mark.parametrize("shape", [(3581, 3580, 100), (3584, 3588, 64), (3585, 3584, 36), (3500, 3600, 4), (3841, 3332, 232),
                                   (1000, 1000, 1000), (2000, 1996, 200), (100, 36, 8), (70, 2044, 52), (1, 4, 4),
                                   (4300, 4348, 100), (4090, 5116, 68)])
def test_wave_tile_ragged_edges(prism, oracle, shape):
    """M, N, K that are not whole tiles, N and K multiples of 4: with enough 256 x 256 tiles for the CUs
    (the first five shapes) the whole-tile kernel, for small problems the one-wave-per-tile kernel
    (64 x 64 or 32 x 32 tiles, at least four K tiles of 16, those beyond K all zeros), both with
    zero-filled edges; the last two shapes have 289 and 320 tiles for 256 CUs, so the ragged tiles of
    the partial second round are cut into one-wave tiles (32 x 32 and 64 x 64), pieces outside C included (rows beyond a matrix arrive as zeros through the buffer
    descriptor's range check, columns beyond N and k beyond K through an out-of-range lane offset).
    A and B sit between NaNs, so one element read from outside a matrix, or from the next row, would
    poison the output; C is fenced against stores outside it. Every element is checked, with and
    without reading C."""
    M, N, K = shape
    A, B, Cm = oracle.gen_sgemm(M, N, K, seed=M + 3 * K)
    for beta in (0.5, 0.0):
        buf = torch.full((M * N + 512,), 777.0, dtype=torch.float32, device=DEV)
        c = buf[256:256 + M * N].view(M, N)
        c.copy_(dev(Cm))
        prism.sgemm(M, N, K, 1.25, nan_fenced(A), nan_fenced(B), beta, c, variant=5)
        out = host(buf)
        assert np.all(out[:256] == 777.0) and np.all(out[256 + M * N:] == 777.0)
        got = out[256:256 + M * N].reshape(M, N)
        assert np.max(np.abs(got - oracle.np_sgemm_f64(1.25, A, B, beta, Cm))) <= tol(oracle, K, A, B, beta, Cm)


@pytest.mark.parametrize("shape", [(2304, 2304, 64), (2560, 2816, 48), (2300, 2564, 100), (2817, 2560, 36),
                                   (3072, 3072, 64), (3328, 2944, 32), (3000, 3332, 68), (3329, 3072, 20), (1152, 6144, 16),
                                   (2080, 2048, 128), (2270, 2500, 200), (2048, 2048, 96), (1920, 2040, 100), (1664, 2048, 33)])
def test_wave_tile_mid_sizes(prism, oracle, shape):
    """Between the one-wave tiles (up to 1024 tiles of 64 x 64) and the 256 x 256 tiles (from 192 of them): the
    direct-to-LDS kernel on 128 x 256 tiles when those give nearly every CU one (2817 x 2560: 230 tiles), else
    on 64 x 256 tiles, whose partial last round is cut into one-wave tiles of 32 x 32 when K is at least 64 and
    that is cheaper (2304^2: 68 of 324 tiles, 3072^2: 64 of 576, 2080 x 2048: 8 of 264, 2270 x 2500: 104 of 360,
    the last with zero-filled edges); the last three shapes have 192 to 256 tiles of 64 x 256, a single round,
    which is taken in place of one-wave tiles (whole, with edges, with rows that are not 16 B aligned); whole and
    ragged shapes, K tile counts from 1 up. Operands between NaNs, C fenced, every element checked, with and without reading C."""
    M, N, K = shape
    A, B, Cm = oracle.gen_sgemm(M, N, K, seed=M + 5 * K)
    for beta in (0.5, 0.0):
        buf = torch.full((M * N + 512,), 777.0, dtype=torch.float32, device=DEV)
        c = buf[256:256 + M * N].view(M, N)
        c.copy_(dev(Cm))
        prism.sgemm(M, N, K, 1.25, nan_fenced(A), nan_fenced(B), beta, c, variant=5)
        out = host(buf)
        assert np.all(out[:256] == 777.0) and np.all(out[256 + M * N:] == 777.0)
        got = out[256:256 + M * N].reshape(M, N)
        assert np.max(np.abs(got - oracle.np_sgemm_f64(1.25, A, B, beta, Cm))) <= tol(oracle, K, A, B, beta, Cm)


@pytest.mark.parametrize("shape", [(3581, 3582, 101), (3584, 3585, 67), (3585, 3587, 38), (3500, 3601, 5), (3841, 3333, 233),
                                   (3584, 3584, 7), (3584, 3584, 64), (2300, 2566, 101), (3001, 3333, 69), (2304, 2305, 4),
                                   (4300, 4349, 101), (4090, 5117, 70), (5377, 5375, 66),
                                   (1001, 1001, 1001), (2001, 1999, 130), (64, 65, 6), (33, 31, 4), (700, 130, 77),
                                   (2305, 2303, 70)])
def test_wave_tile_rows_not_16_byte_aligned(prism, oracle, shape):
    """N or K not a multiple of 4, or matrices that start at an odd element: rows are then only 4 B aligned and
    the direct-to-LDS kernel runs in its ragged form (256 x 256 tiles for the first seven shapes, 128 x 256 and
    64 x 256 tiles for the next three; the last three have 289, 320 and 462 tiles for 256 CUs, so the 33, 64 and
    206 tiles of their partial last round are cut into 64 x 256 slices, or not at all; the last five are small
    problems for the one-wave-per-tile kernel's ragged form, 64 x 64 and 32 x 32 tiles, K tile counts from 1 up, and the
    last has 333 tiles of 64 x 256 for 256 CUs, whose last 77 are cut into ragged one-wave tiles of 32 x 32): 16 B loads from 4 B-aligned addresses, a K loop over K rounded down to a
    multiple of 4 with the last K % 4 values added in front of the write-back, and C written element by element
    where a chunk straddles N. A and B sit between NaNs and C is fenced; every element is checked, with and
    without reading C, with the matrices at an even and at an odd element."""
    M, N, K = shape
    A, B, Cm = oracle.gen_sgemm(M, N, K, seed=M + 7 * K)
    for beta, start, c_at in ((0.5, 1024, 256), (0.0, 1021, 255), (0.5, 1022, 257)):
        buf = torch.full((M * N + 512,), 777.0, dtype=torch.float32, device=DEV)
        c = buf[c_at:c_at + M * N].view(M, N)
        c.copy_(dev(Cm))
        prism.sgemm(M, N, K, 1.25, nan_fenced(A, start), nan_fenced(B, start), beta, c, variant=5)
        out = host(buf)
        assert np.all(out[:c_at] == 777.0) and np.all(out[c_at + M * N:] == 777.0)
        got = out[c_at:c_at + M * N].reshape(M, N)
        assert np.max(np.abs(got - oracle.np_sgemm_f64(1.25, A, B, beta, Cm))) <= tol(oracle, K, A, B, beta, Cm)


def test_wave_tile_ragged_rows_keep_infinities_in_their_row(prism, oracle):
    """An infinite element of A belongs to one row of C only. With K % 4 != 0 the 16 B chunk that holds the
    end of row r of A also holds the head of row r + 1; the ragged form must not let that reach row r
    (0 x inf would turn it into NaN). Likewise an infinite element in the first column of B stays in column 0."""
    M, N, K = 3584, 3585, 67
    A, B, Cm = oracle.gen_sgemm(M, N, K, seed=11)
    A[1000, 0] = np.inf
    B[5, 0] = np.inf
    c = dev(Cm).clone()
    prism.sgemm(M, N, K, 1.0, dev(A), dev(B), 0.0, c, variant=5)
    got = host(c)
    clean = np.ones((M, N), dtype=bool)
    clean[1000, :] = False
    clean[:, 0] = False
    assert np.all(np.isfinite(got[clean]))
    assert not np.any(np.isfinite(got[1000, :])) and not np.any(np.isfinite(got[:, 0]))
    A[1000, 0] = 0.0
    B[5, 0] = 0.0
    want = oracle.np_sgemm_f64(1.0, A, B, 0.0, Cm)
    assert np.max(np.abs(got[clean] - want[clean])) <= tol(oracle, K, A, B, 0.0, Cm)


def test_wave_tile_ragged_tall_matrix(prism, oracle):
    """A ragged A of more than 4 GiB: the bytes from a tile's first row to the end of A do not fit the 32 bits
    of a buffer descriptor's extent and are cut to 2 GiB - 1 (a tile only reaches 256 rows ahead). Rows are
    sampled from the first and last tiles and from the tile whose remaining byte count is smallest modulo
    2^32, where an extent that wrapped around instead would zero-fill rows that exist."""
    M, N, K = 1_100_003, 260, 1000
    g = torch.Generator(device=DEV)
    g.manual_seed(1)
    A = torch.rand((M, K), dtype=torch.float32, device=DEV, generator=g) * 2 - 1
    B = torch.rand((K, N), dtype=torch.float32, device=DEV, generator=g) * 2 - 1
    C = torch.full((M, N), 3.0, dtype=torch.float32, device=DEV)
    prism.sgemm(M, N, K, 1.0, A, B, 0.0, C, variant=5)
    torch.cuda.synchronize()
    left = [(M - 256 * t) * K * 4 for t in range((M + 255) // 256)]
    worst = min((t for t in range(len(left)) if left[t] >= 2**32), key=lambda t: left[t] % 2**32)
    assert left[worst] % 2**32 < 256 * K * 4  # a wrapped extent would end inside this tile
    rows = np.unique(np.concatenate([np.arange(0, 256, 37), np.arange(worst * 256, worst * 256 + 256, 5),
                                     np.arange(M - 300, M, 7)]))
    it = torch.from_numpy(rows).to(DEV)
    want = A[it].cpu().numpy().astype(np.float64) @ B.cpu().numpy().astype(np.float64)
    got = C[it].cpu().numpy()
    assert np.max(np.abs(got - want)) <= 1e-5 * np.sqrt(K)


def _device_inputs(M, N, K):
    g = torch.Generator(device=DEV)
    g.manual_seed(0)
    A = torch.rand((M, K), dtype=torch.float32, device=DEV, generator=g) * 2 - 1
    B = torch.rand((K, N), dtype=torch.float32, device=DEV, generator=g) * 2 - 1
    C0 = torch.rand((M, N), dtype=torch.float32, device=DEV, generator=g) * 2 - 1
    return A, B, C0


def _bound(K, beta):
    # entries are uniform in [-1, 1): max|A| max|B| <= 1; the beta * C term adds its own rounding
    return 1e-5 * np.sqrt(K) + (abs(beta) * 2**-22 if beta else 0.0)


def _full_check(prism, M, N, K, alpha, beta, variant, linearity=True):
    """Full-size run; EVERY element is compared with an fp64 product formed on the device
    (fp64_referee.sgemm_max_err_fp64: torch's fp64 GEMM on row blocks), bound 1e-5 * sqrt(K) * max|A| * max|B|."""
    import fp64_referee
    A, B, C0 = _device_inputs(M, N, K)
    c = C0.clone()
    prism.sgemm(M, N, K, alpha, A, B, beta, c, variant=variant)
    err = fp64_referee.sgemm_max_err_fp64(alpha, A, B, beta, C0, c)
    assert err <= _bound(K, beta), f"kernel {variant} {M}x{N}x{K}: max error {err:.3e}"
    if linearity:  # doubling alpha with beta = 0 doubles every element exactly
        c1 = torch.empty_like(c)
        c2 = torch.empty_like(c)
        prism.sgemm(M, N, K, 1.0, A, B, 0.0, c1, variant=variant)
        prism.sgemm(M, N, K, 2.0, A, B, 0.0, c2, variant=variant)
        assert torch.equal(c2, 2.0 * c1)
    return c


@pytest.mark.parametrize("n", [4096, 8192])
def test_baseline_square_all_kernels_full_size(prism, oracle, n):
    """BASELINE's square sizes 4096 and 8192 (alpha 1, beta 0.5) for every kernel of the progression: every
    element against the fp64 product, and kernels 1, 2, 3, 4, 6 (one fused multiply-add per k, in order)
    bit-identical to each other. The device-side fp64 product that judges them is itself compared with the
    CPU oracle on 32 sampled rows of the same problem."""
    import fp64_referee
    A, B, C0 = _device_inputs(n, n, n)
    assert fp64_referee.pin_sgemm_referee(oracle, 1.0, A, B, 0.5, C0) <= 1e-9
    del A, B, C0
    first = None
    for v in ALL:
        c = _full_check(prism, n, n, n, 1.0, 0.5, v, linearity=(v == 5))
        if v in EXACT:
            first = c if first is None else first
            assert torch.equal(c, first), f"kernel {v} differs from kernel 1 bitwise at n = {n}"


def test_wave_tile_16384x16384x512(prism):
    _full_check(prism, 16384, 16384, 512, 1.0, 0.0, 5)


@pytest.mark.parametrize("shape", [(4096, 4096, 128), (128, 4096, 4096), (8191, 4097, 1023), (16384, 16384, 512)])
def test_baseline_tail_shapes_all_kernels_full(prism, oracle, shape):
    """BASELINE's non-square and tail shapes (beta = 0) through every kernel, every element against fp64
    (the device product pinned to the CPU oracle on sampled rows first)."""
    import fp64_referee
    M, N, K = shape
    A, B, C0 = _device_inputs(M, N, K)
    assert fp64_referee.pin_sgemm_referee(oracle, 1.0, A, B, 0.0, C0) <= 1e-9
    del A, B, C0
    for v in ALL:
        _full_check(prism, M, N, K, 1.0, 0.0, v, linearity=False)
