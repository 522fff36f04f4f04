"""Pins the CPU oracle (oracle/prism_oracle.c) before anything is compared with it.

The reference holds no numeric golden vectors for this path, so every oracle
function is pinned by what the mathematics fixes: closed forms, hand-computed
wrap/rounding cases, invariants, brute force in exact arithmetic, and library
routines that compute the same thing another way (numpy.cumsum, numpy float64
matmul, torch's bfloat16 cast). Each check is chosen so that a plausible slip
(dropped term, wrong index, transposed operand, wrong rounding) fails it.
"""
from fractions import Fraction

import numpy as np
import pytest


# ------------------------------------------------------------------- add_m --

def test_add_m_hand_cases(oracle):
    x = np.array([0, 1, -1, 2**31 - 1, 2**31 - 7, 2**31 - 8, -2**31], dtype=np.int32)
    y = oracle.add_m(x, 7)
    # computed by hand: INT_MAX + 7 wraps to INT_MIN + 6, INT_MAX - 6 + 7 wraps to INT_MIN
    assert y.tolist() == [7, 8, 6, -2**31 + 6, -2**31, 2**31 - 1, -2**31 + 7]
    assert oracle.add_m(x, -1).tolist() == [-1, 0, -2, 2**31 - 2, 2**31 - 8, 2**31 - 9, 2**31 - 1]


def test_add_m_matches_wide_arithmetic(oracle):
    x = oracle.gen_add_m(100_000, seed=1)
    for m in (7, -7, 2**31 - 1, -2**31, 0):
        assert np.array_equal(oracle.add_m(x, m), oracle.np_add_m(x, m))
    # inverse: adding m then -m is the identity even through wrap-around
    assert np.array_equal(oracle.add_m(oracle.add_m(x, 2**31 - 1), -(2**31 - 1)), x)


# -------------------------------------------------------------------- scan --

def test_scan_closed_forms(oracle):
    ones = np.ones(70_000, dtype=np.int32)
    assert np.array_equal(oracle.scan_cpu(ones), np.arange(1, 70_001, dtype=np.int32))
    # 1..n -> triangular numbers (exact in int64, reduced mod 2^32)
    n = 100_000
    x = np.arange(1, n + 1, dtype=np.int64)
    tri = (x * (x + 1) // 2) % 2**32
    assert np.array_equal(oracle.scan_cpu(x.astype(np.uint32)), tri.astype(np.uint32))
    # alternating +a, -a returns to zero at every even position
    alt = np.tile(np.array([123456789, -123456789], dtype=np.int32), 500)
    out = oracle.scan_cpu(alt)
    assert np.all(out[1::2] == 0) and np.all(out[0::2] == 123456789)


def test_scan_wraps_like_uint32(oracle):
    x = np.full(10, 2**31 - 1, dtype=np.int32)
    expect = [((2**31 - 1) * (i + 1)) % 2**32 for i in range(10)]
    assert oracle.scan_cpu(x).view(np.uint32).tolist() == expect
    assert oracle.scan_cpu(np.array([], dtype=np.int32)).size == 0
    assert oracle.scan_cpu(np.array([-5], dtype=np.int32)).tolist() == [-5]


def test_exclusive_scan_closed_forms_and_relation_to_inclusive(oracle):
    ones = np.ones(70_000, dtype=np.int32)
    assert np.array_equal(oracle.scan_exclusive_cpu(ones), np.arange(0, 70_000, dtype=np.int32))
    x = np.full(6, 2**31 - 1, dtype=np.int32)  # wraps at the third element
    assert oracle.scan_exclusive_cpu(x).view(np.uint32).tolist() == [((2**31 - 1) * i) % 2**32 for i in range(6)]
    assert oracle.scan_exclusive_cpu(np.array([], dtype=np.int32)).size == 0
    assert oracle.scan_exclusive_cpu(np.array([-5], dtype=np.int32)).tolist() == [0]
    for n in (1, 2, 63, 64, 65, 4097, 100_003):
        x = oracle.gen_scan(n, seed=n)
        ex = oracle.scan_exclusive_cpu(x)
        inc = np.cumsum(x, dtype=np.int32)
        assert ex[0] == 0 and np.array_equal(ex[1:], inc[:-1])                        # shifted inclusive sums
        assert np.array_equal(ex.view(np.uint32) + x.view(np.uint32), inc.view(np.uint32))  # exclusive + element


def test_running_maximum_closed_forms_library_routine_and_invariants(oracle):
    rising = np.arange(-40_000, 40_000, dtype=np.int32)
    assert np.array_equal(oracle.scan_max_cpu(rising), rising)
    assert np.all(oracle.scan_max_cpu(rising[::-1].copy()) == 39_999)
    lo, hi = np.iinfo(np.int32).min, np.iinfo(np.int32).max
    assert oracle.scan_max_cpu(np.array([lo, lo, -7, lo, hi, 3], dtype=np.int32)).tolist() == [lo, lo, -7, -7, hi, hi]
    assert oracle.scan_max_cpu(np.array([], dtype=np.int32)).size == 0
    for n in (1, 2, 63, 64, 65, 4097, 100_003):
        x = np.random.default_rng(n).integers(lo, hi, n, dtype=np.int32, endpoint=True)
        got = oracle.scan_max_cpu(x)
        assert np.array_equal(got, np.maximum.accumulate(x))
        assert np.all(np.diff(got.astype(np.int64)) >= 0) and np.all(got >= x)
        steps = np.flatnonzero(np.diff(got.astype(np.int64)) > 0) + 1
        assert got[0] == x[0] and np.array_equal(got[steps], x[steps])  # a new maximum is the element itself


def test_segmented_scan_special_cases_hand_case_and_two_library_routes(oracle):
    """Pins oracle_segmented_scan_cpu: without heads it is the plain scan; with every element a head it is the
    input; a hand-computed case with a wrap; against numpy.cumsum run segment by segment; and against the
    closed form through ONE global cumulative sum (out[i] = S[i] - S[start(i) - 1])."""
    rng = np.random.default_rng(5)
    x = rng.integers(-1000, 1001, 10_000, dtype=np.int32)
    none = np.zeros(x.size, np.uint8)
    assert np.array_equal(oracle.segmented_scan_cpu(x, none), oracle.scan_cpu(x))
    assert np.array_equal(oracle.segmented_scan_cpu(x, np.ones(x.size, np.uint8)), x)
    hx = np.array([5, 7, 2**31 - 1, 1, 4, -3, 10], dtype=np.int32)
    hh = np.array([0, 0, 1, 0, 0, 255, 0], dtype=np.uint8)  # element 0 starts a segment whatever its flag says
    assert oracle.segmented_scan_cpu(hx, hh).tolist() == [5, 12, 2**31 - 1, -2**31, -2**31 + 4, -3, 7]
    for mean in (1.5, 7, 300, 5000):
        h = oracle.gen_heads(x.size, mean, seed=int(mean))
        got = oracle.segmented_scan_cpu(x, h)
        want = np.empty_like(x)
        starts = np.flatnonzero(np.concatenate([[True], h[1:] != 0]))
        for a, b in zip(starts, np.concatenate([starts[1:], [x.size]])):
            want[a:b] = np.cumsum(x[a:b], dtype=np.int32)
        assert np.array_equal(got, want)
        assert np.array_equal(got, oracle.np_segmented_scan(x, h))
    big = np.full(100, 2**31 - 1, dtype=np.int32)
    bh = np.zeros(100, np.uint8)
    bh[50] = 1
    assert np.array_equal(oracle.segmented_scan_cpu(big, bh), oracle.np_segmented_scan(big, bh))
    assert oracle.segmented_scan_cpu(np.zeros(0, np.int32), np.zeros(0, np.uint8)).size == 0


def test_scan_i64_closed_forms_and_numpy(oracle):
    n = 5000
    assert np.array_equal(oracle.scan_i64_cpu(np.ones(n, np.int64)), np.arange(1, n + 1, dtype=np.int64))
    wrap = np.array([2**63 - 1, 1, 2**63 - 1, 2], dtype=np.int64)
    assert oracle.scan_i64_cpu(wrap).tolist() == [2**63 - 1, -2**63, -1, 1]
    x = np.random.default_rng(6).integers(-2**62, 2**62, 20_000, dtype=np.int64)
    with np.errstate(over="ignore"):
        assert np.array_equal(oracle.scan_i64_cpu(x), np.cumsum(x, dtype=np.int64))
    u = x.view(np.uint64)
    assert np.array_equal(oracle.scan_i64_cpu(u), np.cumsum(u, dtype=np.uint64))


def test_scan_vs_numpy_cumsum_and_difference_invariant(oracle):
    for n in (1, 63, 64, 65, 4095, 4096, 4097, 16384, 100_003):
        x = oracle.gen_scan(n, seed=n)
        out = oracle.scan_cpu(x)
        assert np.array_equal(out, np.cumsum(x, dtype=np.int32))
        assert out[0] == x[0]
        assert np.array_equal((out[1:].view(np.uint32) - out[:-1].view(np.uint32)), x[1:].view(np.uint32))


@pytest.mark.parametrize("n", [16384, 32768, 1 << 20])
@pytest.mark.parametrize("stall", [0, 1, 3, 64])
def test_scan_lookback_restatement_equals_serial(oracle, n, stall):
    """The block-structured algorithm of examples/scan.py gives the serial result on the
    reference's own test sizes and distribution, whatever the look-back depth."""
    x = oracle.gen_scan_reference_style(n)
    assert np.array_equal(oracle.scan_lookback(x, stall), oracle.scan_cpu(x))
    xs = oracle.gen_scan(n, seed=3)
    assert np.array_equal(oracle.scan_lookback(xs, stall), oracle.scan_cpu(xs))


def test_scan_lookback_drops_tail_like_reference_launcher(oracle):
    # block_cnt = n / 16384 (evals/4090_scan/main.cu:73): the last 100 elements are never touched
    x = oracle.gen_scan(16384 * 2 + 100, seed=5)
    out = oracle.scan_lookback(x)
    assert np.array_equal(out[: 16384 * 2], oracle.scan_cpu(x[: 16384 * 2]))
    assert np.array_equal(out[16384 * 2:], x[16384 * 2:])
    short = oracle.gen_scan(1000, seed=6)
    assert np.array_equal(oracle.scan_lookback(short), short)


# ------------------------------------------------------------------- sgemm --

def _exact_sgemm(alpha, A, B, beta, Cm):
    M, K = A.shape
    N = B.shape[1]
    out = [[None] * N for _ in range(M)]
    for i in range(M):
        for j in range(N):
            s = sum(Fraction(float(A[i, k])) * Fraction(float(B[k, j])) for k in range(K))
            out[i][j] = Fraction(float(alpha)) * s + (Fraction(float(beta)) * Fraction(float(Cm[i, j])) if beta != 0 else 0)
    return out


def test_sgemm_fma_exact_on_small_integers(oracle):
    """With small integer entries every fma is exact, so the fp32 oracle must equal the
    rational triple loop. A transposed operand or a wrong stride changes the answer."""
    rng = np.random.default_rng(0)
    M, N, K = 5, 7, 6
    A = rng.integers(-8, 9, (M, K)).astype(np.float32)
    B = rng.integers(-8, 9, (K, N)).astype(np.float32)
    Cm = rng.integers(-8, 9, (M, N)).astype(np.float32)
    got = oracle.sgemm_fma(2.0, A, B, -3.0, Cm)
    want = _exact_sgemm(2.0, A, B, -3.0, Cm)
    for i in range(M):
        for j in range(N):
            assert Fraction(float(got[i, j])) == want[i][j]
    got64 = oracle.sgemm_f64(2.0, A, B, -3.0, Cm)
    for i in range(M):
        for j in range(N):
            assert Fraction(float(got64[i, j])) == want[i][j]


def test_sgemm_special_cases(oracle):
    A, B, Cm = oracle.gen_sgemm(17, 13, 17, seed=2)
    eye = np.eye(17, dtype=np.float32)
    # B = I, alpha = 1, beta = 0: C = A exactly (products with 0 and 1 are exact)
    assert np.array_equal(oracle.sgemm_fma(1.0, A, eye, 0.0, np.zeros((17, 17), np.float32)), A)
    # alpha = 0: C = beta * C exactly (fma(0, acc, beta*c))
    assert np.array_equal(oracle.sgemm_fma(0.0, A, B, 0.5, Cm), np.float32(0.5) * Cm)
    # beta = 0 never reads C: NaN in C must not come through
    poison = np.full((17, 13), np.nan, dtype=np.float32)
    assert np.isfinite(oracle.sgemm_fma(1.0, A, B, 0.0, poison)).all()
    assert np.isfinite(oracle.sgemm_f64(1.0, A, B, 0.0, None)).all()
    # K = 1: outer product
    a, b = A[:, :1].copy(), B[:1, :].copy()
    assert np.array_equal(oracle.sgemm_fma(1.0, a, b, 0.0, poison), a * b)
    # K = 0: C = beta * C
    assert np.array_equal(oracle.sgemm_fma(1.0, np.zeros((17, 0), np.float32), np.zeros((0, 13), np.float32), 2.0, Cm), 2.0 * Cm)


@pytest.mark.parametrize("shape", [(33, 47, 29), (128, 96, 200), (1, 1, 1)])
def test_sgemm_f64_vs_numpy_matmul(oracle, shape):
    M, N, K = shape
    A, B, Cm = oracle.gen_sgemm(M, N, K, seed=M)
    ref = oracle.np_sgemm_f64(0.5, A, B, 3.0, Cm)
    got = oracle.sgemm_f64(0.5, A, B, 3.0, Cm)
    assert np.max(np.abs(got - ref)) <= 1e-12 * max(1, K)
    # the fp32-fma oracle sits inside the documented tolerance of the fp64 one
    fma = oracle.sgemm_fma(0.5, A, B, 3.0, Cm)
    assert np.max(np.abs(fma - ref)) <= 0.5 * oracle.sgemm_tolerance(K, A, B) + 3.0 * 2**-23


# --------------------------------------------------------------- bf16 gemm --

def test_bf16_rounding_hand_cases(oracle):
    L = oracle.lib()
    f = lambda bits: np.array([bits], dtype=np.uint32).view(np.float32)[0]
    assert L.oracle_f32_to_bf16(f(0x3F800000)) == 0x3F80          # 1.0
    assert L.oracle_f32_to_bf16(f(0x3F808000)) == 0x3F80          # tie, low bit even -> down
    assert L.oracle_f32_to_bf16(f(0x3F818000)) == 0x3F82          # tie, low bit odd -> up
    assert L.oracle_f32_to_bf16(f(0x3F808001)) == 0x3F81          # just above the tie -> up
    assert L.oracle_f32_to_bf16(f(0x3F807FFF)) == 0x3F80          # just below the tie -> down
    assert L.oracle_f32_to_bf16(f(0x7F7FFFFF)) == 0x7F80          # FLT_MAX rounds to +inf
    assert L.oracle_f32_to_bf16(f(0xFF800000)) == 0xFF80          # -inf
    assert L.oracle_f32_to_bf16(f(0x7FC00001)) & 0x7FC0 == 0x7FC0  # NaN stays NaN
    assert L.oracle_f32_to_bf16(f(0x7F800001)) & 0x7FFF > 0x7F80   # signalling NaN does not become inf
    assert L.oracle_f32_to_bf16(f(0x80000000)) == 0x8000          # -0


def test_bf16_rounding_vs_torch_and_numpy(oracle):
    torch = pytest.importorskip("torch")
    x = np.random.default_rng(4).standard_normal(200_000).astype(np.float32)
    x[:4] = [0.0, -0.0, 1e-40, 3.0e38]
    got = oracle.f32_to_bf16(x)
    assert np.array_equal(got, oracle.np_f32_to_bf16(x))
    t = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, t)
    # widening is exact and inverse on representable values
    assert np.array_equal(oracle.f32_to_bf16(oracle.bf16_to_f32(got)), got)


def test_gemm_bf16_f64_vs_numpy(oracle):
    for (M, N, K) in [(40, 24, 75), (1, 1, 1), (64, 64, 128)]:
        A16, B16 = oracle.gen_gemm_bf16(M, N, K, seed=K)
        got = oracle.gemm_bf16_f64(A16, B16)
        ref = oracle.np_gemm_bf16_f64(A16, B16)
        assert got.shape == (M, N)
        assert np.max(np.abs(got - ref)) <= 1e-12 * K
    # operand layout: B is N x K (K contiguous); a K x N reading would fail this
    A16 = oracle.np_f32_to_bf16(np.array([[1, 2, 3]], dtype=np.float32))
    B16 = oracle.np_f32_to_bf16(np.array([[1, 0, 0], [0, 1, 0], [1, 1, 1], [0, 0, 2]], dtype=np.float32))
    assert oracle.gemm_bf16_f64(A16, B16).tolist() == [[1.0, 2.0, 6.0, 6.0]]


# ----------------------------------------------------------------- fixtures --

def test_oracle_reproduces_committed_fixtures(oracle, golden):
    x = golden["add_m_x"]
    for m, y in zip(golden["add_m_m"], golden["add_m_y"]):
        assert np.array_equal(oracle.add_m(x, int(m)), y)
    assert np.array_equal(oracle.scan_cpu(golden["scan_x"]), golden["scan_out"])
    assert np.array_equal(np.cumsum(golden["scan_x"], dtype=np.int32), golden["scan_out"])
    assert np.array_equal(oracle.scan_cpu(golden["scan_ref_x"]), golden["scan_ref_out"])
    assert np.array_equal(oracle.scan_lookback(golden["scan_ref_x"]), golden["scan_ref_out"])
    assert np.array_equal(oracle.scan_cpu(golden["scan_wrap_x"]), golden["scan_wrap_out"])
    a, b = (float(v) for v in golden["sgemm_alpha_beta"])
    assert np.array_equal(oracle.sgemm_fma(a, golden["sgemm_A"], golden["sgemm_B"], b, golden["sgemm_C"]),
                          golden["sgemm_out_fma"])
    assert np.allclose(oracle.np_sgemm_f64(a, golden["sgemm_A"], golden["sgemm_B"], b, golden["sgemm_C"]),
                       golden["sgemm_out_f64"], rtol=0, atol=1e-12)
    assert np.allclose(oracle.np_gemm_bf16_f64(golden["bf16_A"], golden["bf16_B"]), golden["bf16_D_f64"],
                       rtol=0, atol=1e-10)
