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


@pytest.mark.parametrize("items", [1, 2, 4, 8, 16])
def test_wave_regroup_blocked_and_striped(prism, items):
    """The wave64 warp_load / warp_store primitives through prism_wave_regroup_i32: blocked -> striped is the
    transpose of every chunk seen as a 64 x items matrix, striped -> blocked its inverse; a partial last chunk
    counts as one padded with zeros; nothing is read or written beyond n."""
    for n in (64 * items * 5, 64 * items * 1000 + 64 * items // 2 + 3, 7, 1 << 20):
        x = np.random.default_rng(n).integers(-2**31, 2**31 - 1, n, dtype=np.int32)
        chunk = 64 * items
        whole = n // chunk * chunk
        want = x.copy()
        want[:whole] = x[:whole].reshape(-1, 64, items).transpose(0, 2, 1).reshape(-1)
        tail = n - whole
        if tail:  # the partial chunk counts as one padded with zeros: position N l + j goes to 64 j + l if that exists
            src = np.arange(tail)
            dst = 64 * (src % items) + src // items
            ok = dst < tail
            want[whole:] = 0
            want[whole + dst[ok]] = x[whole + src[ok]]
        out = torch.full((n + 8,), -7, dtype=torch.int32, device=DEV)
        prism.wave_regroup(dev(x), items, True, out[:n])
        got = host(out)
        assert np.array_equal(got[:n], want) and np.all(got[n:] == -7), (n, items)
        back = prism.wave_regroup(dev(want[:whole]), items, False)
        assert np.array_equal(host(back), x[:whole])
    with pytest.raises(ValueError):
        prism.wave_regroup(torch.zeros(64, dtype=torch.int32, device=DEV), 3)


def test_calibration_streams(prism):
    """The benchmark's calibration kernels (tests/native/calibrate_stream.hip): both copy shapes copy exactly
    `bytes` bytes and nothing more; the one-way kinds run; bad arguments are refused."""
    import calibrate_stream
    lib = calibrate_stream.load()
    n = (1 << 22) + 1024 * 3 + 4  # not a whole number of either kind's workgroups
    x = torch.randint(-2**31, 2**31 - 1, (n + 64,), dtype=torch.int32, device=DEV)
    for kind in (0, 1):
        y = torch.full((n + 64,), 12345, dtype=torch.int32, device=DEV)
        assert lib.calibrate_stream(kind, x.data_ptr(), y.data_ptr(), 4 * n, None) == 0
        torch.cuda.synchronize()
        assert torch.equal(y[:n], x[:n]) and bool((y[n:] == 12345).all()), kind
    y = torch.zeros(n, dtype=torch.int32, device=DEV)
    assert lib.calibrate_stream(2, x.data_ptr(), y.data_ptr(), 4 * n, None) == 0
    assert lib.calibrate_stream(3, None, y.data_ptr(), 4 * n, None) == 0
    torch.cuda.synchronize()
    assert int(y[4]) == 1 and int(y[5]) == 1 and int(y[6]) == 2 and int(y[7]) == 3  # packet 1 = {1, 1, 2, 3}
    assert lib.calibrate_stream(4, x.data_ptr(), y.data_ptr(), 64, None) == 1
    assert lib.calibrate_stream(0, x.data_ptr(), y.data_ptr(), 60, None) == 1
    assert lib.calibrate_stream(0, x[1:].data_ptr(), y.data_ptr(), 64, None) == 1


# -------------------------------------------------------------------- scan --

def test_scan_fixtures(prism, golden):
    for xk, ok in (("scan_x", "scan_out"), ("scan_ref_x", "scan_ref_out"), ("scan_wrap_x", "scan_wrap_out")):
        x = golden[xk]
        xd = dev(x.view(np.int32))
        out = prism.scan(xd)
        assert np.array_equal(host(out).view(x.dtype), golden[ok]), xk


TILE_EDGES = [1, 2, 63, 64, 65, 255, 256, 257, 1023, 1024, 1025, 4095, 4096, 4097, 8191, 8192, 8193,
              16383, 16384, 16385, 32768, 65535, 65536, 65537, 100_003, 262_145,
              1 << 23, (1 << 23) + 1, (1 << 24) - 1, (1 << 24) + 1, (1 << 24) + 65536 * 3 + 5,
              65536 * 300 - 1, 65536 * 300, 65536 * 300 + 1]


@pytest.mark.parametrize("n", TILE_EDGES)
def test_scan_tile_boundaries(prism, oracle, n):
    x = oracle.gen_scan(n, seed=n)
    out = torch.full((n + 8,), -7, dtype=torch.int32, device=DEV)
    prism.scan(dev(x), out[:n])
    got = host(out)
    assert np.array_equal(got[:n], oracle.scan_cpu(x))
    assert np.all(got[n:] == -7)


@pytest.mark.parametrize("n", [1, 2, 255, 256, 257, 4096, 16385, 65536, 65537, 100_003, 1 << 23, (1 << 23) + 1, (1 << 24) - 1, (1 << 24) + 65536 * 3 + 5,
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


@pytest.mark.parametrize("n", [1, 2, 255, 256, 257, 4096, 16385, 65536, 65537, 100_003, 1 << 23, (1 << 23) + 1, (1 << 24) - 1, (1 << 24) + 65536 * 3 + 5,
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
    ws.fill_(0xAB)  # garbage: this launcher clears the workspace itself, like the reference's
    ret = prism.launch_scan(n, xd, ws)
    assert ret.data_ptr() == xd.data_ptr()
    assert np.array_equal(host(xd).view(np.uint32), oracle.scan_cpu(x))


@pytest.mark.parametrize("n", [1 << 20, 1 << 24, 1 << 28])
def test_scan_baseline_sizes(prism, oracle, n):
    x = oracle.gen_scan(n, seed=0)
    out = prism.scan(dev(x))
    assert np.array_equal(host(out), oracle.scan_cpu(x))


@pytest.mark.parametrize("n", [1, 4097, 65536 * 3 + 5, (1 << 24) + 1, 1 << 26, (1 << 28) + 12345])
def test_scan_ticket_order_matches_dispatch_order(prism, oracle, n):
    """Tiles numbered by the ticket counter (the reference's get_block_idx_from_global_counter,
    examples/scan.py:88-99) and tiles numbered by workgroup id give the same bits, also when the two
    orders alternate on one workspace (the ticket counter is back at zero after every call)."""
    x = oracle.gen_scan(n, seed=n % 1000)
    want = oracle.scan_cpu(x)
    xd = dev(x)
    ws = prism.new_scan_workspace(n)
    for ticket in (True, False, True, True, False):
        out = prism.scan(xd, workspace=ws, ticket_order=ticket)
        assert np.array_equal(host(out), want), ticket


def test_scan_that_stops_waiting_helps_its_predecessors(prism, oracle):
    """With the spin limit forced to 0 no look-back waits: a predecessor that has not published when it is polled
    is helped at once, i.e. wave 0 of the waiting tile forms that tile's sum from the input. Every tile then
    finishes on its own, so the bits must be exact whatever the tiles' timing: both tile shapes, 16 B- and 4
    B-aligned views, inclusive, exclusive and running maximum, workgroup-id and ticket order, and IN PLACE, where
    a helped predecessor may be turning its input into output meanwhile (the helper's second poll decides).
    Nothing is reported, and the workspace serves ordinary calls in between."""
    for n in ((1 << 22) + 77, (1 << 26) + 65536 * 5 + 3):
        x = oracle.gen_scan(n, seed=n % 1000)
        inc, exc, mx = oracle.scan_cpu(x), oracle.scan_exclusive_cpu(x), oracle.scan_max_cpu(x)
        xd = dev(x)
        ws = prism.new_scan_workspace(n)
        out = torch.empty_like(xd)
        for kw, want in (({}, inc), ({"ticket_order": True}, inc), ({"exclusive": True}, exc), ({"op": "max"}, mx)):
            print(f"scan n={n} spin_limit=0 {kw}", flush=True)
            prism.scan(xd, out, ws, spin_limit=0, **kw)
            assert np.array_equal(host(out), want), kw
            prism.scan(xd, out, ws, **kw)
            assert np.array_equal(host(out), want), kw
        for _ in range(3):  # in place
            buf = xd.clone()
            prism.scan(buf, buf, ws, spin_limit=0)
            assert np.array_equal(host(buf), inc)
        view_in, view_out = dev(np.concatenate([[5], x]).astype(np.int32))[1:], torch.empty(n + 3, dtype=torch.int32, device=DEV)[3:]
        prism.scan(view_in, view_out, ws, spin_limit=0)  # 4-byte-aligned views: the small tile, element-wise loads
        assert np.array_equal(host(view_out), inc)
        prism.scan_status(ws)


def test_scan_without_helping_that_gives_up_is_an_error(prism, oracle):
    """The plain bounded wait (help=False, PRISM_SCAN_NO_HELP) with the spin limit forced to 0: every look-back
    gives up before it has waited at all. The kernel must still finish (the point of the bound), and the failure
    must be loud: scan() raises, and so does scan_status() after an unchecked call. Afterwards the same workspace
    serves exact scans again and reports nothing."""
    n = 1 << 26
    x = oracle.gen_scan(n, seed=3)
    want = oracle.scan_cpu(x)
    xd = dev(x)
    out = torch.empty_like(xd)
    ws = prism.new_scan_workspace(n)
    for ticket in (True, False):
        with pytest.raises(prism.ScanOrderError, match="gave up waiting"):
            prism.scan(xd, out, ws, ticket_order=ticket, spin_limit=0, help=False)
        prism.scan(xd, out, ws, ticket_order=ticket, spin_limit=0, help=False, check=False)  # asynchronous, unchecked
        with pytest.raises(prism.ScanOrderError):
            prism.scan_status(ws)
        prism.scan_status(ws)  # the report was consumed and the workspace re-initialised
        for _ in range(2):
            prism.scan(xd, out, ws, ticket_order=ticket)
            assert np.array_equal(host(out), want)
    # the reference-shaped launcher checks as well (through the library: no spin limit to force here)
    prism.launch_scan(n, xd, ws)
    assert np.array_equal(host(xd), want)


def test_scan_on_a_workspace_that_was_never_initialised_is_an_error(prism, oracle):
    """A workspace straight from the allocator (here: filled with 0xFF, and once with zeros, which is not the
    initial state either): every kind of scan must leave it alone, exit normally and be reported by
    scan_status() as PRISM_ERROR_SCAN_WORKSPACE; the status call initialises the workspace, after which the same
    buffer serves exact scans."""
    n = (1 << 24) + 5
    x = oracle.gen_scan(n, seed=9)
    want = oracle.scan_cpu(x)
    xd = dev(x)
    out = torch.empty_like(xd)
    heads = torch.zeros(n, dtype=torch.uint8, device=DEV)
    for fill in (0xFF, 0x00):
        ws = torch.full((prism.get_workspace_size(n) + 64,), fill, dtype=torch.uint8, device=DEV)[:prism.get_workspace_size(n)]
        runs = (lambda: prism.scan(xd, out, ws, check=False), lambda: prism.scan(xd, out, ws, check=False, ticket_order=True),
                lambda: prism.segmented_scan(xd, heads, out, ws, check=False),
                lambda: prism.scan(xd.to(torch.int64), None, ws, check=False))
        for run in runs:
            ws.fill_(fill)
            print(f"scan on a workspace filled with {fill:#x}", flush=True)
            run()
            torch.cuda.synchronize()
            body = ws[32:]  # nothing but the report word of the header was written
            assert bool((body == fill).all())
            with pytest.raises(prism.ScanWorkspaceError, match="not initialised"):
                prism.scan_status(ws)
            prism.scan_status(ws)
            prism.scan(xd, out, ws)
            assert np.array_equal(host(out), want)


def test_scan_while_another_stream_keeps_the_gpu_busy(prism, oracle):
    """Scans of 2^28 elements while a second stream (default priority) runs long SGEMMs that compete for every
    CU: workgroups of the scan then start whenever the other kernel leaves room, in no particular rhythm.
    The bits must be exact and nothing may be reported, in workgroup-id order (the default) and in ticket order."""
    n = 1 << 28
    g = torch.Generator(device=DEV)
    g.manual_seed(0)
    xd = torch.randint(-1000, 1001, (n,), dtype=torch.int32, device=DEV, generator=g)
    out = torch.empty_like(xd)
    ws = prism.new_scan_workspace(n)
    prism.scan(xd, out, ws)
    want = out.clone()
    assert int(want[-1]) == ((int(xd.sum(dtype=torch.int64)) + 2**31) % 2**32) - 2**31
    assert bool(torch.equal(want[1:] - want[:-1], xd[1:]))
    M = 4096
    A = torch.rand((M, M), device=DEV)
    B = torch.rand((M, M), device=DEV)
    C = torch.zeros((M, M), device=DEV)
    side = torch.cuda.Stream()  # default priority
    torch.cuda.synchronize()
    for ticket in (False, True):
        with torch.cuda.stream(side):
            for variant in (3, 6, 3, 6, 3, 6):  # 7 ms and 2 ms apiece: about 30 ms of competing work
                prism.sgemm(M, M, M, 1.0, A, B, 0.0, C, variant=variant)
        for rep in range(12):
            out.zero_()
            print(f"scan 2^28 beside SGEMMs on another stream, ticket_order={ticket}, repeat {rep}", flush=True)
            prism.scan(xd, out, ws, ticket_order=ticket, check=False)
        prism.scan_status(ws)
        assert torch.equal(out, want)
        side.synchronize()
        prism.scan(xd, out, ws, ticket_order=ticket)
        assert torch.equal(out, want)


def test_scan_workspace_shared_by_calls_of_any_length_and_kind(prism, oracle):
    """One workspace, initialised once, then calls of very different tile counts and kinds back to back
    and unsynchronised: every call clears the status words the call before it used (also those of a longer
    call), so no call may see a stale word. Long, short and long again is the case that needs the
    high-water mark in the header."""
    big, mid, small = (1 << 26) + 77, (1 << 22) + 5, 70_001
    ws = prism.new_scan_workspace(big)
    xs = {n: oracle.gen_scan(n, seed=n % 97) for n in (big, mid, small)}
    xd = {n: dev(x) for n, x in xs.items()}
    inc = {n: oracle.scan_cpu(x) for n, x in xs.items()}
    plan = [(big, {}), (small, {}), (big, {}), (small, {}), (small, {}), (big, {"ticket_order": True}),
            (mid, {"exclusive": True}), (small, {"op": "max"}), (mid, {}), (big, {"exclusive": True}),
            (small, {"ticket_order": True}), (small, {}), (small, {}), (big, {}), (mid, {"op": "min"}), (big, {})]
    outs = []
    for n, kw in plan:  # all enqueued before anything is checked
        outs.append(prism.scan(xd[n], workspace=ws, check=False, **kw))
    prism.scan_status(ws)
    for (n, kw), out in zip(plan, outs):
        x = xs[n]
        if kw.get("exclusive"):
            want = oracle.scan_exclusive_cpu(x)
        elif kw.get("op") == "max":
            want = oracle.scan_max_cpu(x)
        elif kw.get("op") == "min":
            want = ~oracle.scan_max_cpu(~x)
        else:
            want = inc[n]
        assert np.array_equal(host(out), want), (n, kw)


SEG_SIZES = [1, 2, 63, 64, 65, 255, 256, 257, 1023, 1025, 4096, 16383, 16384, 16385, 65535, 65536, 65537, 100_003,
             262_145, 1 << 23, (1 << 23) + 1, (1 << 24) - 1, (1 << 24) + 65536 * 3 + 5, 1 << 26]


@pytest.mark.parametrize("n", SEG_SIZES)
def test_segmented_scan(prism, oracle, n):
    """Sums that start again at every head, on both tile shapes, for segments that are much shorter than a
    packet, about a wave's row, about a tile and many tiles long, with no head at all and with every element a
    head; out of place with a fenced output, in place, from views that are only 4-byte (values) / 1-byte
    (heads) aligned, and through one workspace shared with plain scans. Bit for bit against the serial loop."""
    x = oracle.gen_scan(n, seed=n % 101)
    xd = dev(x)
    ws = prism.new_scan_workspace(n)
    for mean in (1.3, 6, 300, 20_000, 3_000_000):
        h = oracle.gen_heads(n, mean, seed=int(mean) + n % 7)
        want = oracle.segmented_scan_cpu(x, h)
        out = torch.full((n + 8,), -7, dtype=torch.int32, device=DEV)
        prism.segmented_scan(xd, dev(h), out[:n], workspace=ws)
        got = host(out)
        assert np.array_equal(got[:n], want), mean
        assert np.all(got[n:] == -7)
        assert np.array_equal(host(prism.scan(xd, workspace=ws)), oracle.scan_cpu(x))  # same workspace, other kind
    none, every = np.zeros(n, np.uint8), np.ones(n, np.uint8)
    assert np.array_equal(host(prism.segmented_scan(xd, dev(none), workspace=ws)), oracle.scan_cpu(x))
    assert np.array_equal(host(prism.segmented_scan(xd, dev(every), workspace=ws)), x)
    h = oracle.gen_heads(n, 50, seed=3)
    want = oracle.segmented_scan_cpu(x, h)
    buf = xd.clone()
    prism.segmented_scan(buf, dev(h).bool(), buf, workspace=ws)  # in place, bool flags
    assert np.array_equal(host(buf), want)
    if n >= 256:
        x1 = dev(np.concatenate([[0], x]).astype(np.int32))[1:]
        h1 = dev(np.concatenate([[9], h]).astype(np.uint8))[1:]
        y = torch.zeros(n + 1, dtype=torch.int32, device=DEV)
        prism.segmented_scan(x1, h1, y[1:], workspace=ws)
        assert np.array_equal(host(y)[1:], want)
        prism.segmented_scan(xd, h1, buf, workspace=ws)  # aligned values, unaligned heads
        assert np.array_equal(host(buf), want)


def test_segmented_scan_2pow30_properties(prism):
    """Full size: out[i] == in[i] at every head, out[i] - out[i-1] == in[i] everywhere else, over the whole
    array, for segments of about 1000 elements and for one head in the middle of every 2^20."""
    n = 1 << 30
    g = torch.Generator(device=DEV)
    g.manual_seed(1)
    x = torch.randint(-1000, 1001, (n,), dtype=torch.int32, device=DEV, generator=g)
    for kind in ("dense", "sparse"):
        if kind == "dense":
            heads = (torch.rand((n,), device=DEV, generator=g) < 1e-3).to(torch.uint8)
        else:
            heads = torch.zeros(n, dtype=torch.uint8, device=DEV)
            heads[(1 << 19)::(1 << 20)] = 1
        out = prism.segmented_scan(x, heads)
        chunk = 1 << 26
        assert int(out[0]) == int(x[0])
        for s in range(0, n, chunk):
            e = s + chunk
            lo = max(s, 1)
            is_head = heads[lo:e] != 0
            want = torch.where(is_head, x[lo:e], out[lo - 1:e - 1] + x[lo:e])
            assert torch.equal(out[lo:e], want), (kind, s)
        del out


@pytest.mark.parametrize("n", [1, 2, 127, 128, 129, 4095, 32767, 32768, 32769, 65536, 100_003, 1 << 20, (1 << 22) + 32768 * 3 + 5, 1 << 26])
def test_scan_of_64_bit_elements(prism, oracle, n):
    """Inclusive sums modulo 2^64: values that use all 64 bits (so both status halves matter and carries cross
    them), out of place with a fenced output, in place, as uint64, from a view that is only 8-byte aligned, and on
    a workspace shared with 32-bit scans. Bit for bit against the serial loop."""
    rng = np.random.default_rng(n % 211)
    x = rng.integers(-2**62, 2**62, n, dtype=np.int64)
    want = oracle.scan_i64_cpu(x)
    ws = prism.new_scan_workspace(n)
    xd = dev(x)
    out = torch.full((n + 8,), -7, dtype=torch.int64, device=DEV)
    prism.scan(xd, out[:n], workspace=ws)
    got = host(out)
    assert np.array_equal(got[:n], want) and np.all(got[n:] == -7)
    small = oracle.gen_scan(min(n, 70_001), seed=1)
    assert np.array_equal(host(prism.scan(dev(small), workspace=ws)), oracle.scan_cpu(small))  # a 32-bit scan in between
    buf = xd.clone()
    prism.scan(buf, buf, workspace=ws)
    assert np.array_equal(host(buf), want)
    carries = np.full(n, 0xffffffff, dtype=np.uint64)  # every addition carries into the high half
    got_u = host(prism.scan(dev(carries.view(np.int64)), workspace=ws)).view(np.uint64)
    assert np.array_equal(got_u, oracle.scan_i64_cpu(carries))
    if n >= 128:
        x1 = dev(np.concatenate([[0], x]).astype(np.int64))[1:]
        y = torch.zeros(n + 1, dtype=torch.int64, device=DEV)
        prism.scan(x1, y[1:], workspace=ws)
        assert np.array_equal(host(y)[1:], want)
    with pytest.raises(ValueError):
        prism.scan(xd, exclusive=True)


def test_scan_of_64_bit_elements_2pow29_properties(prism):
    """4 GiB in, 4 GiB out: difference invariant over the whole array and the last element against block sums."""
    n = 1 << 29
    g = torch.Generator(device=DEV)
    g.manual_seed(2)
    x = torch.randint(-2**40, 2**40, (n,), dtype=torch.int64, device=DEV, generator=g)
    out = prism.scan(x)
    assert int(out[0]) == int(x[0])
    chunk = 1 << 25
    total = 0
    for s in range(0, n, chunk):
        e = s + chunk
        lo = max(s, 1)
        assert torch.equal(out[lo:e] - out[lo - 1:e - 1], x[lo:e])
        total += int(x[s:e].sum())
    assert int(out[-1]) == ((total + 2**63) % 2**64) - 2**63


def test_segmented_and_64_bit_scans_help_their_predecessors_too(prism, oracle):
    """The spin limit forced to 0, as in test_scan_that_stops_waiting_helps_its_predecessors, for the other two
    kinds of scan. Segmented: the helper forms a tile's (head seen, sum) pair from its input and head bytes, for
    segments much shorter than a tile (nearly every tile holds a head and ends the walk), about a tile long and
    many tiles long (walks across helped, flagless tiles), none at all; both tile shapes, unaligned views, in
    place. 64-bit: values that use all 64 bits, both alignments, in place. Bit for bit against the serial loops;
    nothing is reported, and without helping the same calls are errors."""
    for n in ((1 << 22) + 77, (1 << 25) + 65536 * 5 + 3):
        x = oracle.gen_scan(n, seed=n % 1000)
        xd = dev(x)
        ws = prism.new_scan_workspace(n)
        for mean in (6, 40_000, 3_000_000):
            h = oracle.gen_heads(n, mean, seed=int(mean) % 97)
            hd = dev(h)
            want = oracle.segmented_scan_cpu(x, h)
            print(f"segmented scan n={n} mean segment {mean} spin_limit=0", flush=True)
            out = prism.segmented_scan(xd, hd, workspace=ws, spin_limit=0)
            assert np.array_equal(host(out), want), mean
            buf = xd.clone()
            prism.segmented_scan(buf, hd, buf, workspace=ws, spin_limit=0)  # in place
            assert np.array_equal(host(buf), want), mean
        assert np.array_equal(host(prism.segmented_scan(xd, dev(np.zeros(n, np.uint8)), workspace=ws, spin_limit=0)), oracle.scan_cpu(x))
        h = oracle.gen_heads(n, 500, seed=5)
        x1 = dev(np.concatenate([[0], x]).astype(np.int32))[1:]
        h1 = dev(np.concatenate([[9], h]).astype(np.uint8))[1:]
        y = torch.zeros(n + 1, dtype=torch.int32, device=DEV)
        prism.segmented_scan(x1, h1, y[1:], workspace=ws, spin_limit=0)  # element-wise loads, the small tile
        assert np.array_equal(host(y)[1:], oracle.segmented_scan_cpu(x, h))
        with pytest.raises(prism.ScanOrderError, match="gave up waiting"):
            prism.segmented_scan(xd, dev(np.zeros(n, np.uint8)), workspace=ws, spin_limit=0, help=False)
        assert np.array_equal(host(prism.segmented_scan(xd, dev(h), workspace=ws)), oracle.segmented_scan_cpu(x, h))

        rng = np.random.default_rng(n % 211)
        m = n // 2
        x64 = rng.integers(-2**62, 2**62, m, dtype=np.int64)
        want64 = oracle.scan_i64_cpu(x64)
        x64d = dev(x64)
        print(f"64-bit scan n={m} spin_limit=0", flush=True)
        assert np.array_equal(host(prism.scan(x64d, workspace=ws, spin_limit=0)), want64)
        for _ in range(2):
            buf = x64d.clone()
            prism.scan(buf, buf, workspace=ws, spin_limit=0)
            assert np.array_equal(host(buf), want64)
        x1 = dev(np.concatenate([[0], x64]).astype(np.int64))[1:]
        y = torch.zeros(m + 1, dtype=torch.int64, device=DEV)
        prism.scan(x1, y[1:], workspace=ws, spin_limit=0)  # 8-byte-aligned views
        assert np.array_equal(host(y)[1:], want64)
        with pytest.raises(prism.ScanOrderError, match="gave up waiting"):
            prism.scan(x64d, workspace=ws, spin_limit=0, help=False)
        assert np.array_equal(host(prism.scan(x64d, workspace=ws)), want64)
        prism.scan_status(ws)


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
    ws = prism.new_scan_workspace(1 << 20)
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
