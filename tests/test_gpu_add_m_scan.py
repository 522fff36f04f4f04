"""GPU parity tests for add_m and the look-back scan: the HIP kernels, called through
the C ABI, against the CPU oracle on identical seeded inputs. Bit-exact."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def dev(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def host(t: torch.Tensor) -> np.ndarray:
    torch.cuda.synchronize()
    return t.cpu().numpy()


# ------------------------------------------------------------------- add_m --

def test_add_m_fixture(prism, golden):
    x = dev(golden["add_m_x"])
    for m, want in zip(golden["add_m_m"], golden["add_m_y"]):
        y = torch.empty_like(x)
        prism.add_m(x, y, int(m))
        assert np.array_equal(host(y), want)


@pytest.mark.parametrize("n", [1, 3, 4, 5, 255, 1023, 1024, 1025, 4099, 1 << 20, (1 << 20) + 3])
def test_add_m_ragged_sizes(prism, oracle, n):
    x = oracle.gen_add_m(n, seed=n)
    y = torch.full((n + 8,), 12345, dtype=torch.int32, device=DEV)
    prism.add_m(dev(x), y[:n], 7)
    got = host(y)
    assert np.array_equal(got[:n], oracle.add_m(x, 7))
    assert np.all(got[n:] == 12345)  # nothing written past n


def test_add_m_baseline_config_and_inplace(prism, oracle):
    # BASELINE config: n = 2^24, x in [-2^20, 2^20), m = 7
    n = 1 << 24
    x = oracle.gen_add_m(n, seed=0)
    xd = dev(x)
    y = torch.empty_like(xd)
    prism.add_m(xd, y, 7)
    want = oracle.add_m(x, 7)
    assert np.array_equal(host(y), want)
    prism.add_m(xd, xd, 7)  # x == y is allowed
    assert np.array_equal(host(xd), want)


def test_add_m_unaligned_views_and_wrap(prism, oracle):
    base = oracle.gen_add_m(10_007, seed=9)
    base[:3] = [2**31 - 1, -2**31, 2**31 - 7]
    buf = dev(base)
    out = torch.zeros(10_010, dtype=torch.int32, device=DEV)
    # element offsets 1 and 3 make both pointers 4-byte but not 16-byte aligned
    prism.add_m(buf[1:], out[3:3 + 10_006], 2**31 - 1)
    assert np.array_equal(host(out)[3:3 + 10_006], oracle.add_m(base[1:], 2**31 - 1))
    assert host(out)[:3].tolist() == [0, 0, 0]


# -------------------------------------------------------------------- scan --

def test_scan_fixtures(prism, golden):
    for xk, ok in (("scan_x", "scan_out"), ("scan_ref_x", "scan_ref_out"), ("scan_wrap_x", "scan_wrap_out")):
        x = golden[xk]
        xd = dev(x.view(np.int32))
        out = prism.scan(xd)
        assert np.array_equal(host(out).view(x.dtype), golden[ok]), xk


TILE_EDGES = [1, 2, 63, 64, 65, 255, 256, 257, 1023, 1024, 1025, 4095, 4096, 4097, 8191, 8192, 8193,
              16383, 16384, 16385, 32768, 65535, 65536, 65537, 100_003, 262_145,
              (1 << 24) - 1, (1 << 24) + 1, (1 << 24) + 65536 * 3 + 5,
              65536 * 300 - 1, 65536 * 300, 65536 * 300 + 1]


@pytest.mark.parametrize("n", TILE_EDGES)
def test_scan_tile_boundaries(prism, oracle, n):
    x = oracle.gen_scan(n, seed=n)
    out = torch.full((n + 8,), -7, dtype=torch.int32, device=DEV)
    prism.scan(dev(x), out[:n])
    got = host(out)
    assert np.array_equal(got[:n], oracle.scan_cpu(x))
    assert np.all(got[n:] == -7)


@pytest.mark.parametrize("n", [1, 2, 255, 256, 257, 4096, 16385, 65536, 65537, 100_003, (1 << 24) - 1, (1 << 24) + 65536 * 3 + 5,
                               1 << 26])
def test_exclusive_scan(prism, oracle, n):
    """The exclusive form (out[0] = 0, out[i] = in[0] + ... + in[i-1]) on both tile shapes, out of place with a
    fenced output and in place; and exclusive + element == inclusive, element for element."""
    x = oracle.gen_scan(n, seed=n + 1)
    want = oracle.scan_exclusive_cpu(x)
    out = torch.full((n + 8,), -7, dtype=torch.int32, device=DEV)
    xd = dev(x)
    prism.scan(xd, out[:n], exclusive=True)
    got = host(out)
    assert np.array_equal(got[:n], want) and np.all(got[n:] == -7)
    assert np.array_equal(got[:n].view(np.uint32) + x.view(np.uint32), host(prism.scan(xd)).view(np.uint32))
    prism.scan(xd, xd, exclusive=True)
    assert np.array_equal(host(xd), want)
    if n >= 256:  # only 4 B aligned views take the scalar path
        y = torch.zeros(n + 1, dtype=torch.int32, device=DEV)
        prism.scan(dev(np.concatenate([[0], x]).astype(np.int32))[1:], y[1:], exclusive=True)
        assert np.array_equal(host(y)[1:], want)


@pytest.mark.parametrize("n", [1, 2, 255, 256, 257, 4096, 16385, 65536, 65537, 100_003, (1 << 24) - 1, (1 << 24) + 65536 * 3 + 5,
                               1 << 26])
def test_running_maximum(prism, oracle, n):
    """The operator form of the scan, out[i] = max(in[0..i]) over int32, on both tile shapes: out of place with a
    fenced output, in place, and from a view that is only 4 B aligned (the scalar path). Three inputs: uniform
    over all of int32 (new maxima die out quickly), a slow random walk (new maxima throughout, so every stage
    of the kernel carries a value that matters), and all INT32_MIN (the operator's identity as data)."""
    lo, hi = np.iinfo(np.int32).min, np.iinfo(np.int32).max
    rng = np.random.default_rng(n + 2)
    walk = np.cumsum(rng.integers(-3, 4, n, dtype=np.int64)).clip(lo, hi).astype(np.int32)
    for x in (rng.integers(lo, hi, n, dtype=np.int32, endpoint=True), walk, np.full(n, lo, dtype=np.int32)):
        want = oracle.scan_max_cpu(x)
        out = torch.full((n + 8,), -7, dtype=torch.int32, device=DEV)
        xd = dev(x)
        prism.scan(xd, out[:n], op="max")
        got = host(out)
        assert np.array_equal(got[:n], want) and np.all(got[n:] == -7)
        prism.scan(xd, xd, op="max")
        assert np.array_equal(host(xd), want)
        if n >= 256:
            y = torch.zeros(n + 1, dtype=torch.int32, device=DEV)
            prism.scan(dev(np.concatenate([[0], x]).astype(np.int32))[1:], y[1:], op="max")
            assert np.array_equal(host(y)[1:], want)
        # the running minimum is the running maximum of the bitwise complements, complemented (~v = -v - 1
        # reverses the order of int32 without overflow): checked against the same oracle
        prism.scan(dev(~x), out[:n], op="min")
        got = host(out)
        assert np.array_equal(~got[:n], want) and np.all(got[n:] == -7)


@pytest.mark.parametrize("n", [16384, 32768, 1 << 20, 1 << 24, 1 << 26])
def test_scan_reference_test_sizes_inplace(prism, oracle, n):
    """The reference's own correctness sizes and distribution (evals/4090_scan/main.cu:97-109),
    through the reference-shaped launcher: in place, uint32."""
    x = oracle.gen_scan_reference_style(n)
    xd = dev(x.view(np.int32))
    ws = torch.empty(prism.get_workspace_size(n), dtype=torch.uint8, device=DEV)
    ws.fill_(0xAB)  # garbage: the launcher resets the workspace itself
    ret = prism.launch_scan(n, xd, ws)
    assert ret.data_ptr() == xd.data_ptr()
    assert np.array_equal(host(xd).view(np.uint32), oracle.scan_cpu(x))


@pytest.mark.parametrize("n", [1 << 20, 1 << 24, 1 << 28])
def test_scan_baseline_sizes(prism, oracle, n):
    x = oracle.gen_scan(n, seed=0)
    out = prism.scan(dev(x))
    assert np.array_equal(host(out), oracle.scan_cpu(x))


@pytest.fixture
def scan_env(monkeypatch):
    """The library reads PRISM_SCAN_ORDER / PRISM_SCAN_SPIN_LIMIT at every call."""
    def set_(order=None, spin_limit=None):
        for key, val in (("PRISM_SCAN_ORDER", order), ("PRISM_SCAN_SPIN_LIMIT", spin_limit)):
            if val is None:
                monkeypatch.delenv(key, raising=False)
            else:
                monkeypatch.setenv(key, str(val))
    yield set_
    set_()


@pytest.mark.parametrize("n", [1, 4097, 65536 * 3 + 5, (1 << 24) + 1, 1 << 26, (1 << 28) + 12345])
def test_scan_ticket_order_matches_dispatch_order(prism, oracle, scan_env, n):
    """Tiles numbered by the ticket counter (the reference's get_block_idx_from_global_counter,
    examples/scan.py:88-99) and tiles numbered by workgroup id give the same bits."""
    x = oracle.gen_scan(n, seed=n % 1000)
    want = oracle.scan_cpu(x)
    xd = dev(x)
    for order in ("ticket", None):
        scan_env(order=order)
        out = prism.scan(xd)
        assert np.array_equal(host(out), want), order


def test_scan_look_back_wait_is_bounded(prism, oracle, scan_env):
    """With the spin limit forced to 0 a look-back that has to wait even once gives up: the kernel
    must still finish, and a wave that gave up reports its tile + 1 in word 2 of the workspace.
    With the default limit the same workspace reports nothing and the result is exact."""
    n = 1 << 26
    x = oracle.gen_scan(n, seed=3)
    xd = dev(x)
    out = torch.empty_like(xd)
    ws = torch.empty(prism.get_workspace_size(n), dtype=torch.uint8, device=DEV)
    for order in ("ticket", None):
        scan_env(order=order, spin_limit=0)
        prism.scan(xd, out, ws)
        torch.cuda.synchronize()  # the point of the test: this returns
        report = int(ws[8:12].view(torch.int32).item())
        tiles = -(-n // 16384)
        assert 0 <= report <= tiles
        if report == 0:  # nobody had to wait: then the result must be right
            assert np.array_equal(host(out), oracle.scan_cpu(x))
        scan_env(order=order)
        prism.scan(xd, out, ws)
        assert int(ws[8:12].view(torch.int32).item()) == 0
        assert np.array_equal(host(out), oracle.scan_cpu(x))


def test_scan_2pow30_properties(prism):
    """Full BASELINE size (4 GiB in, 4 GiB out): checked on the device through
    size-independent properties - first element, the difference invariant
    out[i] - out[i-1] == in[i] over the whole array, and block sums against int64."""
    n = 1 << 30
    g = torch.Generator(device=DEV)
    g.manual_seed(0)
    x = torch.randint(-1000, 1001, (n,), dtype=torch.int32, device=DEV, generator=g)
    out = prism.scan(x)
    torch.cuda.synchronize()
    assert int(out[0]) == int(x[0])
    chunk = 1 << 26
    running = 0
    for s in range(0, n, chunk):
        e = s + chunk
        o, xi = out[s:e], x[s:e]
        lo = max(s, 1)
        assert torch.equal(out[lo:e] - out[lo - 1:e - 1], x[lo:e])
        running += int(xi.sum(dtype=torch.int64))
        want_last = ((running + 2**31) % 2**32) - 2**31
        assert int(o[-1]) == want_last
    del out
    # in place on the same buffer gives the same bits
    ref_last = want_last
    prism.scan(x, x)
    torch.cuda.synchronize()
    assert int(x[-1]) == ref_last


def test_scan_wraparound_and_all_ones(prism, oracle):
    n = 300_000
    ones = torch.ones(n, dtype=torch.int32, device=DEV)
    assert np.array_equal(host(prism.scan(ones)), np.arange(1, n + 1, dtype=np.int32))
    big = np.full(50_000, 2**31 - 1, dtype=np.int32)
    assert np.array_equal(host(prism.scan(dev(big))), oracle.scan_cpu(big))


def test_scan_workspace_reuse_and_unaligned(prism, oracle):
    n = 70_001
    ws = torch.empty(prism.get_workspace_size(1 << 20), dtype=torch.uint8, device=DEV)
    for seed in range(4):  # same workspace, different data and lengths, back to back
        m = n - 1000 * seed
        x = oracle.gen_scan(m, seed=seed)
        out = prism.scan(dev(x), workspace=ws)
        assert np.array_equal(host(out), oracle.scan_cpu(x))
    for n in (n, (1 << 24) + 12_345):  # small-tile and large-tile kernels
        x = oracle.gen_scan(n + 1, seed=42)
        xd = dev(x)
        out = torch.zeros(n + 3, dtype=torch.int32, device=DEV)
        prism.scan(xd[1:], out[3:3 + n])  # 4-byte-aligned only: scalar path
        assert np.array_equal(host(out)[3:], oracle.scan_cpu(x[1:]))


def test_scan_on_a_side_stream(prism, oracle):
    x = oracle.gen_scan(1 << 20, seed=8)
    xd = dev(x)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        out = prism.scan(xd)
    s.synchronize()
    assert np.array_equal(host(out), oracle.scan_cpu(x))
