"""The HIP emitter for the thread-level subset of the Prism DSL (prism_amd/hipgen.py); kernels with a
block perspective are covered by test_hipgen_blocks.py.

CPU: the text printed for the reference's add_m_thread example (examples/add_m_thread.py:10-19) equals
the text the reference documents for it (README.md:133-140); bounded and launcher forms; constructs
outside the subset are refused by name; the launcher cross-compiles for gfx950.
GPU: the compiled kernel is run through its C launcher and checked bit for bit against numpy.
"""
import ctypes

import numpy as np
import pytest

from prism_amd import hipgen
from prism_amd.hipgen import HipgenError, block, const, generate, generate_launcher, grid, group, partition, prism, ptr, requires, thread


@requires(grid[1], thread[1])
@prism("global")
def add_m_thread(x: ptr(const(int)) @ grid[1],
                 y: ptr(int) @ grid[1],
                 m: int @ grid[1]):
    tid: int @ thread[1] = id()
    with partition(x, p=thread[1], offset=tid) as x_thread:
        with partition(y, p=thread[1], offset=tid) as y_thread:
            with group(thread[1]):
                y_thread[0] = x_thread[0] + m


@requires(grid[1], thread[1])
@prism("global")
def clipped_axpy(x: ptr(const(float)) @ grid[1], y: ptr(float) @ grid[1], a: float @ grid[1], lim: float @ grid[1]):
    """y = min(a * x + y, lim), written with an if."""
    i: int @ thread[1] = id()
    with partition(x, p=thread[1], offset=i) as xv:
        with partition(y, p=thread[1], offset=i) as yv:
            with group(thread[1]):
                t: float @ thread[1] = a * xv[0] + yv[0]
                if t > lim:
                    t = lim
                yv[0] = t


@requires(grid[1], thread[1])
@prism("global")
def block_level(x: ptr(int) @ grid[1]):
    """Declares no block perspective (so it is printed flat) but asks for a block id."""
    bid: int @ block[1] = id()


# README.md:133-140 of the reference: what its generate("add_m_thread") prints.
REFERENCE_TEXT = """__global__ void add_m_thread(const int* x, int* y, int m) {
    int tid = blockIdx.x * blockDim.x + threadIdx.x;
    y[tid] = x[tid] + m;
}
"""


def test_add_m_thread_text_matches_the_reference():
    assert generate("add_m_thread") == REFERENCE_TEXT


def test_bounded_and_launcher_forms():
    text = generate("add_m_thread", bounded=True)
    assert "size_t prism_n" in text.splitlines()[0]
    assert "if (tid >= prism_n) return;" in text
    launcher = generate_launcher("add_m_thread")
    assert 'extern "C" int add_m_thread_launch(const int* x, int* y, int m, size_t n, void* stream)' in launcher
    assert "(n + 255) / 256" in launcher
    with pytest.raises(HipgenError):
        generate_launcher("add_m_thread", block_size=100)


def test_if_and_locals():
    text = generate("clipped_axpy")
    assert "float t = (a * x[i]) + y[i];" in text
    assert "if (t > lim) {" in text and "t = lim;" in text and "y[i] = t;" in text


def test_constructs_outside_the_subset_are_named():
    with pytest.raises(HipgenError, match=r"block\[1\]"):
        generate("block_level")
    with pytest.raises(HipgenError, match="no kernel named"):
        generate("nope")
    with pytest.raises(HipgenError):
        group(thread[1])  # body constructs are parsed, never called


def test_launcher_compiles_for_gfx950(tmp_path):
    lib = hipgen.build("add_m_thread", out_dir=str(tmp_path))
    assert hasattr(lib, "add_m_thread_launch")
    assert (tmp_path / "add_m_thread.hip").read_text().startswith("#include <hip/hip_runtime.h>")


@pytest.fixture(scope="module")
def built(tmp_path_factory):
    """Both example kernels, generated and compiled once for the GPU tests of this module."""
    d = tmp_path_factory.mktemp("hipgen")
    return {name: hipgen.build(name, out_dir=str(d)) for name in ("add_m_thread", "clipped_axpy")}


@pytest.mark.gpu
@pytest.mark.parametrize("n", [1, 255, 256, 257, 1 << 20, (1 << 24), (1 << 24) + 3])
def test_generated_add_m_thread_runs_bit_exact(built, n):
    import torch
    lib = built["add_m_thread"]
    lib.add_m_thread_launch.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t, ctypes.c_void_p]
    rng = np.random.default_rng(n)
    x = rng.integers(-2**20, 2**20, n, dtype=np.int32)
    x[0] = 2**31 - 3  # wraps with m = 7
    xd = torch.from_numpy(x).to("cuda:0")
    yd = torch.full((n + 4,), -1, dtype=torch.int32, device="cuda:0")
    assert lib.add_m_thread_launch(xd.data_ptr(), yd.data_ptr(), 7, n, None) == 0
    torch.cuda.synchronize()
    y = yd.cpu().numpy()
    assert np.array_equal(y[:n], x + np.int32(7))
    assert np.all(y[n:] == -1)


@pytest.mark.gpu
def test_generated_float_kernel_with_branch(built):
    import torch
    lib = built["clipped_axpy"]
    lib.clipped_axpy_launch.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float, ctypes.c_float,
                                        ctypes.c_size_t, ctypes.c_void_p]
    n = 100_003
    rng = np.random.default_rng(0)
    x = rng.standard_normal(n).astype(np.float32)
    y = rng.standard_normal(n).astype(np.float32)
    xd, yd = torch.from_numpy(x).to("cuda:0"), torch.from_numpy(y).to("cuda:0")
    assert lib.clipped_axpy_launch(xd.data_ptr(), yd.data_ptr(), 1.5, 0.25, n, None) == 0
    torch.cuda.synchronize()
    # the compiler may contract a * x + y into one fma: accept either rounding
    plain = np.minimum(np.float32(1.5) * x + y, np.float32(0.25))
    fused = np.minimum((np.float64(1.5) * x.astype(np.float64) + y.astype(np.float64)).astype(np.float32), np.float32(0.25))
    got = yd.cpu().numpy()
    assert np.all((got == plain) | (got == fused))
