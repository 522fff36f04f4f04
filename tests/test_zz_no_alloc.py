"""prism_scan_i32_static: the scan entry point that allocates nothing.

Its status words live in a device array inside the library instead of a caller-allocated workspace. Called
through the C ABI and checked bit for bit against prism_scan_i32 (and the CPU oracle) on two calls in a
row, the second on a smaller input, then on sizes of both tile shapes, in place, and from a view that is
only 4-byte aligned. The file name sorts last on purpose: this test also has to pass after every other
test has used the library, and a failure here must not hide the tests before it.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def test_static_scratch_scan_matches_the_workspace_scan(prism, oracle):
    from prism_amd import _lib
    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream

    def both(x):
        xd = torch.from_numpy(x).to(DEV)
        n = xd.numel()
        got = torch.full((n + 8,), -7, dtype=torch.int32, device=DEV)
        assert lib.prism_scan_i32_static(xd.data_ptr(), got.data_ptr(), n, stream) == 0, _lib.last_error()
        ws = prism.new_scan_workspace(n)
        want = torch.empty_like(xd)
        assert lib.prism_scan_i32(xd.data_ptr(), want.data_ptr(), n, ws.data_ptr(), ws.numel(), stream) == 0
        assert lib.prism_scan_status(None, 0, stream) == 0, _lib.last_error()
        assert lib.prism_scan_status(ws.data_ptr(), ws.numel(), stream) == 0
        assert torch.equal(got[:n], want) and bool((got[n:] == -7).all())
        return got[:n].cpu().numpy()

    # two calls in a row, the second with a smaller input
    big = oracle.gen_scan((1 << 24) + 65536 * 3 + 5, seed=11)
    small = oracle.gen_scan(70_001, seed=12)
    assert np.array_equal(both(big), oracle.scan_cpu(big))
    assert np.array_equal(both(small), oracle.scan_cpu(small))
    # back to a long one (the short call must have cleared the long call's status words), then more shapes
    assert np.array_equal(both(big), oracle.scan_cpu(big))
    for n in (1, 255, 16384, 16385, 65537, 1 << 20, 1 << 23, (1 << 23) + 1, (1 << 24) - 1, 1 << 26):
        x = oracle.gen_scan(n, seed=n % 89)
        assert np.array_equal(both(x), oracle.scan_cpu(x)), n

    # several unsynchronised calls, in place, and 4-byte-aligned views
    x = oracle.gen_scan((1 << 22) + 3, seed=5)
    xd = torch.from_numpy(x).to(DEV)
    for _ in range(5):
        buf = xd.clone()
        assert lib.prism_scan_i32_static(buf.data_ptr(), buf.data_ptr(), buf.numel(), stream) == 0
    assert np.array_equal(buf.cpu().numpy(), oracle.scan_cpu(x))
    out = torch.zeros(x.size + 2, dtype=torch.int32, device=DEV)
    assert lib.prism_scan_i32_static(xd[1:].data_ptr(), out[3:].data_ptr(), x.size - 1, stream) == 0
    assert np.array_equal(out.cpu().numpy()[3:], oracle.scan_cpu(x[1:]))
    assert lib.prism_scan_status(None, 0, stream) == 0

    # nothing is allocated: buffers made beforehand, then calls of both tile shapes; neither PyTorch's allocator
    # nor the device's free memory moves (the first call on this device, which looks the array up, is behind us)
    big_in = torch.from_numpy(big).to(DEV)
    big_out = torch.empty_like(big_in)
    small_in = torch.from_numpy(small).to(DEV)
    small_out = torch.empty_like(small_in)
    torch.cuda.synchronize()
    allocated, reserved, free = torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), torch.cuda.mem_get_info()[0]
    for _ in range(3):
        assert lib.prism_scan_i32_static(big_in.data_ptr(), big_out.data_ptr(), big_in.numel(), stream) == 0
        assert lib.prism_scan_i32_static(small_in.data_ptr(), small_out.data_ptr(), small_in.numel(), stream) == 0
    assert lib.prism_scan_status(None, 0, stream) == 0
    assert (torch.cuda.memory_allocated(), torch.cuda.memory_reserved(), torch.cuda.mem_get_info()[0]) == (allocated, reserved, free)
    assert np.array_equal(big_out.cpu().numpy(), oracle.scan_cpu(big)) and np.array_equal(small_out.cpu().numpy(), oracle.scan_cpu(small))

    # beyond the array's reach: rejected with a clear error, nothing launched
    assert lib.prism_scan_i32_static(xd.data_ptr(), xd.data_ptr(), (1 << 31) + 1, stream) == 1
    assert "2147483648" in _lib.last_error()
    assert lib.prism_scan_i32_static(None, None, 0, stream) == 0


def test_static_scratch_scan_under_graph_capture(prism, oracle):
    """The use the entry point is for: recorded into a HIP graph (no allocation may happen under capture) and
    replayed three times with fresh inputs, eager work and synchronisations in between; every replay against
    the eager result. The set-up call (address look-up and one-time fill) happens before the capture."""
    from prism_amd import _lib
    lib = _lib.load()
    n = (1 << 22) + 12345
    x = torch.zeros(n, dtype=torch.int32, device=DEV)
    out = torch.empty_like(x)
    side = torch.cuda.Stream()  # default priority
    assert lib.prism_scan_status(None, 0, torch.cuda.current_stream().cuda_stream) == 0   # sets the array up
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        assert lib.prism_scan_i32_static(x.data_ptr(), out.data_ptr(), n, side.cuda_stream) == 0
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        assert lib.prism_scan_i32_static(x.data_ptr(), out.data_ptr(), n, torch.cuda.current_stream().cuda_stream) == 0
    for seed in (1, 2, 3):
        xs = oracle.gen_scan(n, seed=seed)
        x.copy_(torch.from_numpy(xs))
        assert lib.prism_scan_i32_static(x.data_ptr(), out.data_ptr(), n, torch.cuda.current_stream().cuda_stream) == 0
        torch.cuda.synchronize()
        eager = out.clone()
        out.fill_(0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager) and np.array_equal(out.cpu().numpy(), oracle.scan_cpu(xs))
    assert lib.prism_scan_status(None, 0, torch.cuda.current_stream().cuda_stream) == 0
