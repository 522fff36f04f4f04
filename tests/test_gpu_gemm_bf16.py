"""GPU parity tests for the bf16 MFMA GEMM (the h100_matmul analogue), through the C ABI.

Oracle: fp64 product of the bf16-rounded inputs. Tolerance (written out here):
  fp32 output   |got - ref| <= 1e-3 * max|ref|            (relative, max-norm)  and
                |got - ref| <= 1e-3 * sum_k |a_k||b_k|    (element-wise, where computed)
  bf16 output   the same plus one bf16 rounding: |got - ref| <= 2^-8 |ref| + 1e-3 * max|ref|
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
REL = 1e-3


def dev16(a16: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a16).view(np.int16)).to(DEV).view(torch.bfloat16)


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def check_f32(oracle, got, A16, B16, ref=None):
    if ref is None:
        ref = oracle.gemm_bf16_f64(A16, B16)
    err = np.abs(got - ref)
    scale = float(np.abs(ref).max(initial=0.0))
    assert err.max(initial=0.0) <= REL * scale + 1e-30
    mag = np.abs(oracle.bf16_to_f32(A16)).astype(np.float64) @ np.abs(oracle.bf16_to_f32(B16)).astype(np.float64).T
    assert np.all(err <= REL * mag + 1e-30)


SHAPES = [(1, 1, 1), (32, 32, 16), (40, 24, 75), (128, 128, 64), (128, 128, 128), (256, 384, 192),
          (130, 200, 72), (64, 64, 8), (100, 36, 1000), (257, 129, 65)]


@pytest.mark.parametrize("shape", SHAPES)
def test_fp32_output_vs_fp64_oracle(prism, oracle, shape):
    M, N, K = shape
    A16, B16 = oracle.gen_gemm_bf16(M, N, K, seed=M * 7 + N + K)
    D = prism.gemm_bf16(dev16(A16), dev16(B16))
    assert D.shape == (M, N) and D.dtype == torch.float32
    check_f32(oracle, host(D), A16, B16)


@pytest.mark.parametrize("shape", [(256, 256, 128), (256, 512, 192), (512, 256, 256), (256, 256, 320), (512, 512, 1024), (256, 256, 384), (256, 256, 448),
                                   (256, 512, 6144), (512, 256, 6208), (128, 384, 6272),
                                   (3072, 3072, 384), (3072, 3072, 192), (2816, 3328, 448), (3072, 3328, 512),
                                   (4352, 4352, 384), (4608, 4608, 384), (2560, 2304, 320), (2304, 2560, 448),
                                   (3072, 3072, 1280), (2048, 4096, 384)])
def test_whole_tile_paths(prism, oracle, shape):
    """Problems made of whole tiles leave the general kernel. Up to 128 tiles of 256 x 256, half the CUs (the first
    ten shapes, the two before the last two, and the last with exactly 128): 128 x 128 tiles, direct-to-LDS ring, four K tiles deep where every CU gets at
    most one tile and K has four tiles (K tile counts of 4, 5, 6, 7, 16, 96, 97 and 98 here), two deep otherwise
    (K of 128 and 192; the two shapes with 360 tiles, the last with 512). From 129 tiles up: an even K tile count from 6 up
    takes the direct-to-LDS pipeline with early fragment reads (6 and 8 K tiles here), the others the
    direct-to-LDS ring of 256 x 256 tiles (3 and 7 K tiles). Two shapes have 289 and 324 tiles for 256 CUs: the 33 or
    68 tiles of the partial second round are cut into 128 x 128 tiles by a second launch (the four-deep ring for
    132 of them, the two-deep ring for 272). In that pipeline the workgroups of XCD x start at K tile 64 x modulo
    the tile count and wrap around: with 6 K tiles at 0, 4, 2, with 20 (the last shape) at 0, 4, 8, 12, 16. Every element is checked, for both
    output types."""
    M, N, K = shape
    A16, B16 = oracle.gen_gemm_bf16(M, N, K, seed=K + M)
    D = prism.gemm_bf16(dev16(A16), dev16(B16))
    ref = oracle.gemm_bf16_f64(A16, B16)
    check_f32(oracle, host(D), A16, B16, ref)
    Cc = torch.full((N * M + 64,), -7.0, dtype=torch.bfloat16, device=DEV)
    prism.runmyh100(M, N, K, dev16(A16), dev16(B16), Cc[32:32 + N * M])
    got = host(Cc.view(torch.int16)).view(np.uint16)
    guard = np.float32(-7.0).view(np.uint32) >> 16
    assert np.all(got[:32] == guard) and np.all(got[32 + N * M:] == guard)
    c = oracle.bf16_to_f32(got[32:32 + N * M]).reshape(N, M).T
    assert np.all(np.abs(c - ref) <= 2.0**-8 * np.abs(ref) + REL * np.abs(ref).max())


@pytest.mark.parametrize("shape", [(3072, 3072, 384), (4352, 4352, 384)])
def test_whole_tiles_with_outputs_at_odd_elements(prism, oracle, shape):
    """Whole tiles write unguarded 16 B packets: fp32 rows in packets of four values, bf16 rows as runs of 16 B that
    went through LDS. The interface asks only element alignment of the outputs, so here D starts at an odd float
    and C at an odd bf16 element, between fences. One launch of one tile per workgroup (144 tiles) and the walking
    launch with a cut partial round (289 tiles)."""
    M, N, K = shape
    A16, B16 = oracle.gen_gemm_bf16(M, N, K, seed=K + 3 * M)
    ref = oracle.gemm_bf16_f64(A16, B16)
    buf = torch.full((M * N + 512,), 777.0, dtype=torch.float32, device=DEV)
    prism.gemm_bf16(dev16(A16), dev16(B16), buf[255:255 + M * N].view(M, N))
    out = host(buf)
    assert np.all(out[:255] == 777.0) and np.all(out[255 + M * N:] == 777.0)
    check_f32(oracle, out[255:255 + M * N].reshape(M, N), A16, B16, ref)
    Cc = torch.full((N * M + 64,), -7.0, dtype=torch.bfloat16, device=DEV)
    prism.runmyh100(M, N, K, dev16(A16), dev16(B16), Cc[31:31 + N * M])
    got = host(Cc.view(torch.int16)).view(np.uint16)
    guard = np.float32(-7.0).view(np.uint32) >> 16
    assert np.all(got[:31] == guard) and np.all(got[31 + N * M:] == guard)
    c = oracle.bf16_to_f32(got[31:31 + N * M]).reshape(N, M).T
    assert np.all(np.abs(c - ref) <= 2.0**-8 * np.abs(ref) + REL * np.abs(ref).max())


def nan_fenced(a16: np.ndarray, start: int = 1024) -> torch.Tensor:
    """The matrix as a view into a device buffer whose other elements are bf16 NaN patterns; `start` is its
    first element's index (a multiple of 8 keeps it 16 B aligned)."""
    buf = torch.full((a16.size + 2048,), 0x7FC0, dtype=torch.int16, device=DEV)
    buf[start:start + a16.size] = torch.from_numpy(np.ascontiguousarray(a16).view(np.int16).ravel()).to(DEV)
    return buf[start:start + a16.size].view(torch.bfloat16).view(a16.shape)


@pytest.mark.parametrize("shape", [(1, 1, 8), (257, 255, 8), (300, 520, 392), (255, 513, 456), (512, 512, 72), (1000, 1000, 1000),
                                   (256, 256, 64), (8, 8, 1032), (264, 24, 6152), (777, 300, 128),
                                   (3000, 3080, 392), (2900, 3100, 72), (3072, 3072, 8), (3000, 3072, 264), (2816, 3000, 328),
                                   (2500, 2300, 264), (3000, 3072, 1288), (4200, 4300, 392), (4600, 4700, 136)])
def test_ragged_shapes_with_aligned_rows(prism, oracle, shape):
    """M, N not whole tiles or K not a multiple of 64, K a multiple of 8: the kernels' edge variants
    (rows beyond the matrix and K tiles beyond K read as zeros through the buffer descriptor's range
    check): the ring of 128 x 128 tiles for small problems (four deep up to 256 tiles with K from 256 up, two
    deep for K below that and for the 360 tiles of the shape before the last), the direct-to-LDS pipeline with early fragment
    reads from 128 tiles of 256 x 256 up (the last shape, 21 K tiles padded to 22 and walked from staggered
    starting points, and the five shapes before the last two: K tile counts of 7, 2, 1, 5 and 6 before
    padding to an even count of at least 4); the last two shapes have 289 and 342 tiles for 256 CUs, whose partial
    second round (33 and 86 tiles) is cut into 128 x 128 edge tiles of the ring, four and two deep. The matrices sit between NaNs, so one element read from outside a
    matrix, or from the next row in the partial K tile, would poison the output; stores are fenced too."""
    check_between_fences(prism, oracle, shape)


@pytest.mark.parametrize("shape", [(2817, 3088, 384), (3072, 3073, 512), (3080, 3072, 640), (4097, 4100, 768), (3088, 2832, 1152),
                                   (2829, 3074, 2048)])
def test_thin_strips_beyond_whole_tiles(prism, oracle, shape):
    """Up to 16 rows and up to 16 columns beyond whole 256 x 256 tiles, over at least half a round of whole tiles, K
    a multiple of 128 from 384 up: the whole tiles run unguarded (one launch, or one workgroup per CU walking
    several tiles in the fourth shape) and the rest as strips, 16 rows of the long operand to a workgroup whose eight
    waves split K (3, 4, 5, 6, 9 and 16 steps of 32 to a wave, with fewer or none for the last waves). fp32 output and the
    transposed bf16 output, where rows and columns change places. Operands and outputs sit between NaNs and
    fences."""
    check_between_fences(prism, oracle, shape)


def check_between_fences(prism, oracle, shape):
    M, N, K = shape
    A16, B16 = oracle.gen_gemm_bf16(M, N, K, seed=3 * M + N + K)
    buf = torch.full((M * N + 512,), 777.0, dtype=torch.float32, device=DEV)
    D = buf[256:256 + M * N].view(M, N)
    prism.gemm_bf16(nan_fenced(A16), nan_fenced(B16), D)
    out = host(buf)
    assert np.all(out[:256] == 777.0) and np.all(out[256 + M * N:] == 777.0)
    ref = oracle.gemm_bf16_f64(A16, B16)
    check_f32(oracle, out[256:256 + M * N].reshape(M, N), A16, B16, ref)
    Cc = torch.full((N * M + 64,), -7.0, dtype=torch.bfloat16, device=DEV)
    prism.runmyh100(M, N, K, nan_fenced(A16), nan_fenced(B16), Cc[32:32 + N * M])
    got = host(Cc.view(torch.int16)).view(np.uint16)
    guard = np.float32(-7.0).view(np.uint32) >> 16
    assert np.all(got[:32] == guard) and np.all(got[32 + N * M:] == guard)
    c = oracle.bf16_to_f32(got[32:32 + N * M]).reshape(N, M).T
    assert np.all(np.abs(c - ref) <= 2.0**-8 * np.abs(ref) + REL * np.abs(ref).max())


@pytest.mark.parametrize("shape", [(3000, 3080, 393), (2900, 3100, 75), (3072, 3072, 9), (3000, 3072, 647), (3072, 3072, 15),
                                   (3072, 3072, 264), (2817, 3001, 406),
                                   (1001, 1001, 1001), (300, 520, 395), (257, 255, 9), (64, 64, 8), (2001, 1999, 130), (1000, 1000, 264),
                                   (4200, 4290, 393), (4700, 4600, 139)])
def test_rows_not_16_byte_aligned(prism, oracle, shape):
    """K not a multiple of 8, or operands that start at an odd element: rows are then only 2 B or 4 B aligned
    and, from 128 tiles of 256 x 256 up, the early-read kernel runs in its ragged form: 16 B direct loads from
    2 B-aligned addresses, a K loop over K rounded down to a multiple of 8 (1 to 11 tiles here, padded to an
    even count of at least 4), and the last K % 8 values of k added on the way out; the six shapes before the last two are
    small problems for the ragged form of the ring of 128 x 128 tiles (two and four deep), and the last two leave a
    partial second round (33 and 86 tiles of 256 x 256) that the same ring finishes. The matrices sit between
    NaNs at an even and at an odd element; stores are fenced; fp32 and bf16 outputs."""
    M, N, K = shape
    A16, B16 = oracle.gen_gemm_bf16(M, N, K, seed=5 * M + N + K)
    ref = oracle.gemm_bf16_f64(A16, B16)
    for start in ((1025, 1030) if K % 8 == 0 else (1024, 1025)):  # K % 8 == 0 at a multiple of 8: the aligned edge variant
        buf = torch.full((M * N + 512,), 777.0, dtype=torch.float32, device=DEV)
        D = buf[255:255 + M * N].view(M, N)
        prism.gemm_bf16(nan_fenced(A16, start), nan_fenced(B16, start), D)
        out = host(buf)
        assert np.all(out[:255] == 777.0) and np.all(out[255 + M * N:] == 777.0)
        check_f32(oracle, out[255:255 + M * N].reshape(M, N), A16, B16, ref)
    Cc = torch.full((N * M + 64,), -7.0, dtype=torch.bfloat16, device=DEV)
    prism.runmyh100(M, N, K, nan_fenced(A16, 1027), nan_fenced(B16, 1029), Cc[31:31 + N * M])
    got = host(Cc.view(torch.int16)).view(np.uint16)
    guard = np.float32(-7.0).view(np.uint32) >> 16
    assert np.all(got[:31] == guard) and np.all(got[31 + N * M:] == guard)
    c = oracle.bf16_to_f32(got[31:31 + N * M]).reshape(N, M).T
    assert np.all(np.abs(c - ref) <= 2.0**-8 * np.abs(ref) + REL * np.abs(ref).max())


def test_fixture(prism, golden, oracle):
    A16, B16 = golden["bf16_A"], golden["bf16_B"]
    D = host(prism.gemm_bf16(dev16(A16), dev16(B16)))
    ref = golden["bf16_D_f64"]
    assert np.max(np.abs(D - ref)) <= REL * np.abs(ref).max()


def test_exact_on_small_integers(prism, oracle):
    """Small integers are exact in bf16 and their dot products exact in fp32: the result must be
    exact whatever the summation order; a wrong operand layout (B read as K x N) fails."""
    rng = np.random.default_rng(2)
    M, N, K = 96, 160, 200
    A = rng.integers(-4, 5, (M, K)).astype(np.float32)
    B = rng.integers(-4, 5, (N, K)).astype(np.float32)
    A16, B16 = oracle.np_f32_to_bf16(A), oracle.np_f32_to_bf16(B)
    D = host(prism.gemm_bf16(dev16(A16), dev16(B16)))
    assert np.array_equal(D, (A.astype(np.float64) @ B.astype(np.float64).T).astype(np.float32))


@pytest.mark.parametrize("shape", [(128, 256, 256), (96, 40, 75), (256, 128, 64)])
def test_runmyh100_layout_and_rounding(prism, oracle, shape):
    """Reference launcher shape: bf16 output, column-major (C[n*M + m])."""
    M, N, K = shape
    A16, B16 = oracle.gen_gemm_bf16(M, N, K, seed=K)
    C = torch.zeros(M * N + 64, dtype=torch.bfloat16, device=DEV)
    prism.runmyh100(M, N, K, dev16(A16), dev16(B16), C[:M * N], None)
    raw = host(C.view(torch.int16)).view(np.uint16)
    assert np.all(raw[M * N:] == 0)
    got = oracle.bf16_to_f32(raw[:M * N]).reshape(N, M).T  # column-major M x N
    ref = oracle.gemm_bf16_f64(A16, B16)
    assert np.all(np.abs(got - ref) <= 2.0**-8 * np.abs(ref) + REL * np.abs(ref).max())
    # identical to rounding the fp32-output kernel's result (same accumulation, different store)
    D = host(prism.gemm_bf16(dev16(A16), dev16(B16)))
    assert np.array_equal(oracle.np_f32_to_bf16(D), raw[:M * N].reshape(N, M).T)


def test_no_write_outside_and_k_zero(prism, oracle):
    M, N, K = 70, 45, 33
    A16, B16 = oracle.gen_gemm_bf16(M, N, K, seed=1)
    buf = torch.full((M * N + 512,), 777.0, dtype=torch.float32, device=DEV)
    D = buf[256:256 + M * N].view(M, N)
    prism.gemm_bf16(dev16(A16), dev16(B16), D)
    out = host(buf)
    assert np.all(out[:256] == 777.0) and np.all(out[256 + M * N:] == 777.0)
    check_f32(oracle, out[256:256 + M * N].reshape(M, N), A16, B16)
    Z = prism.gemm_bf16(torch.zeros((M, 0), dtype=torch.bfloat16, device=DEV),
                        torch.zeros((N, 0), dtype=torch.bfloat16, device=DEV),
                        torch.full((M, N), 5.0, dtype=torch.float32, device=DEV))
    assert np.all(host(Z) == 0.0)


@pytest.mark.parametrize("n", [4096, 8192, 16384])
def test_baseline_sizes_full(prism, oracle, n):
    """BASELINE sizes: N(0,1) inputs rounded to bf16; EVERY element against an fp64 product of the rounded
    inputs formed on the device (fp64_referee.gemm_bf16_max_err_fp64), bound 1e-3 relative to the largest element.
    The device product is itself checked against the CPU oracle on 32 sampled rows."""
    import fp64_referee
    g = torch.Generator(device=DEV)
    g.manual_seed(0)
    A = torch.randn((n, n), dtype=torch.float32, device=DEV, generator=g).to(torch.bfloat16)
    B = torch.randn((n, n), dtype=torch.float32, device=DEV, generator=g).to(torch.bfloat16)
    D = prism.gemm_bf16(A, B)
    err, ref_max = fp64_referee.gemm_bf16_max_err_fp64(A, B, D)
    assert err <= REL * ref_max, f"n = {n}: max error {err:.3e}, largest element {ref_max:.3e}"
    assert fp64_referee.pin_gemm_bf16_referee(oracle, A, B) <= 1e-9
    # scaling an input by 2 (exact in bf16) scales the output exactly
    D2 = prism.gemm_bf16((A.float() * 2).to(torch.bfloat16), B)
    assert torch.equal(D2, 2.0 * D)
