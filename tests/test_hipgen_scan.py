"""The look-back scans of prism_amd/examples/scan.py, generated for gfx950.

CPU: the structure of the generated text (device functions before their callers, where the barriers land).
GPU: bit for bit against numpy's wrapping cumulative sum.
"""
import ctypes

import numpy as np
import pytest

from prism_amd import hipgen
from prism_amd.examples import scan as _programs  # noqa: F401  (defines the kernels)
from prism_amd.hipgen import generate, generate_launcher

def lines(text):
    return [ln.strip() for ln in text.splitlines()]


def test_structure_of_the_generated_scan():
    got = lines(generate("lookback_scan"))
    assert got[0] == ("__global__ void lookback_scan(const uint32_t* x, uint32_t* y, uint32_t* counter, uint64_t* status, "
                      "int spin_limit) {")
    assert "uint32_t tile = take_ticket(__block_id_0, __thread_id_0, __smem, counter);" in got
    assert "__shared__ uint32_t scanned[1024];" in got and "__shared__ uint32_t upto[16];" in got
    assert "int wave = (__thread_id_1 / 64);" in got
    assert "publish(__block_id_1, __thread_id_1, __smem, status_blk, tile, 2, (before + total));" in got
    # barriers: in front of the `if` in which the first wavefront reads the row ends, in front of the read of the
    # total, and none inside a branch; the write-back reads arrays that are complete by then
    sync = [n for n, ln in enumerate(got) if ln == "__syncthreads();"]
    assert len(sync) == 2
    assert got[sync[0] + 1] == "if ((wave == 0)) {" and got[sync[1] + 1] == "uint32_t total = upto[15];"
    launcher = generate_launcher("lookback_scan")
    kernel_at = launcher.index(" lookback_scan(")
    assert all(launcher.index(f" {name}(") < kernel_at for name in ("shift_up_in_wavefront", "take_ticket", "publish", "look_back"))
    assert "__hip_atomic_store(&status[tile]" in launcher and "__shfl_up(val, delta, 64)" in launcher


def test_barriers_of_the_scan_made_of_device_functions():
    """Three calls in a row that are handed LDS arrays: a barrier in front of the second (it reads what the first
    wrote) and in front of the third, none further down: the pointer the third call returns is not followed, and
    the write-back takes `scanned` as a pointer to const, last written two barriers ago. The reference prints its
    scan the same way (generated/scan_kernel.cu:16-26)."""
    got = lines(generate("lookback_scan_by_parts"))
    sync = [n for n, ln in enumerate(got) if ln == "__syncthreads();"]
    assert len(sync) == 2
    assert got[sync[0] - 1] == "__shared__ uint32_t spare[16];"
    assert got[sync[0] + 1] == "collect_row_ends(__block_id_1, __thread_id_1, __smem, scanned, ends);"
    assert got[sync[0] + 2] == "__syncthreads();"
    assert got[sync[1] + 1] == "uint32_t* upto = scan_row_ends(__block_id_1, __thread_id_1, __smem, ends, spare);"
    assert got[sync[1] + 2] == "uint32_t total = upto[15];"
    assert got[-6] == "write_back(__block_id_1, __thread_id_1, __smem, y_tile, scanned, upto, before);"
    # the third function orders its own two arrays: one barrier between writing `spare` and reading it back, one
    # as the last statement of the loop's body, so that its result is complete when it returns
    inner = lines(generate("scan_row_ends"))
    assert inner[0] == ("__device__ uint32_t* scan_row_ends(int __block_id, int __thread_id, char* __smem, uint32_t* ends, "
                        "uint32_t* spare) {")
    at = [n for n, ln in enumerate(inner) if ln == "__syncthreads();"]
    assert len(at) == 2 and inner[at[0] + 1] == "if ((t < 16)) {" and inner[at[1] - 1] == "stride *= 2;" and inner[at[1] + 1] == "}"
    assert "const uint32_t* scanned" in generate("collect_row_ends").splitlines()[0]


def test_structure_of_the_wide_scan():
    """Sixteen elements per thread in a private array; one barrier between the wavefront totals going into LDS and
    the sum that reads them; the look-back reads 64 status words per step."""
    got = lines(generate("lookback_scan_wide"))
    assert "uint32_t v[16];" in got and "v[i] += v[(i - 1)];" in got
    sync = [n for n, ln in enumerate(got) if ln == "__syncthreads();"]
    assert len(sync) == 1 and got[sync[0] + 1].startswith("uint32_t total = (((wave_sums[0] + wave_sums[1])")
    assert "uint32_t base = ((before + earlier_waves) + (upto_me - v[15]));" in got
    text = generate("look_back_wide")
    assert "__ballot((word >> 32) == 2)" in text and "spin_limit" in text


KERNELS = {"lookback_scan": 1024, "lookback_scan_by_parts": 1024, "lookback_scan_wide": 4096, "lookback_scan_striped": 65536}   # kernel -> elements per tile


@pytest.fixture(scope="module")
def built(tmp_path_factory):
    d = tmp_path_factory.mktemp("hipgen_scan")
    from prism_amd import examples
    return {name: hipgen.build(name, out_dir=str(d), block_size=examples.KERNELS[name][1]) for name in KERNELS}


def test_launcher_compiles_for_gfx950(built):
    for name in KERNELS:
        assert hasattr(built[name], f"{name}_launch")


@pytest.mark.gpu
@pytest.mark.parametrize("name", KERNELS)
@pytest.mark.parametrize("tiles", [1, 2, 7, 300, 4096])
def test_generated_lookback_scan_is_bit_exact(built, tiles, name):
    import torch
    fn = getattr(built[name], f"{name}_launch")
    fn.argtypes = [ctypes.c_void_p] * 4 + [ctypes.c_int, ctypes.c_uint, ctypes.c_void_p]
    tiles = min(tiles, (1 << 26) // KERNELS[name])   # at most 2^26 elements: the host check is a numpy cumsum
    n = tiles * KERNELS[name]
    x = np.random.default_rng(tiles).integers(0, 2**32, n, dtype=np.uint32)
    xd = torch.from_numpy(x.view(np.int32)).to("cuda:0")
    yd = torch.full((n + 8,), -5, dtype=torch.int32, device="cuda:0")
    counter = torch.zeros(1, dtype=torch.int32, device="cuda:0")
    status = torch.zeros(tiles, dtype=torch.int64, device="cuda:0")
    torch.cuda.synchronize()
    assert fn(xd.data_ptr(), yd.data_ptr(), counter.data_ptr(), status.data_ptr(), 1 << 22, tiles, None) == 0
    torch.cuda.synchronize()
    y = yd.cpu().numpy().view(np.uint32)
    assert np.array_equal(y[:n], np.cumsum(x, dtype=np.uint32)) and np.all(y[n:] == np.uint32(2**32 - 5))
    assert int(counter.item()) == tiles
