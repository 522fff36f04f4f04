"""A single-pass prefix sum with decoupled look-back, written in the Prism surface syntax and generated for gfx950.

The program follows the decomposition of the reference's scan example (examples/scan.py: a ticket from a global
counter :88-99, row scans by lane shifts :106-128, the scan of the row ends :147-173, aggregate / prefix records
and the look-back in target text :34-85, the write-back with the tile's prefix :176-193), on 64-lane wavefronts:
a tile is 1024 elements = 16 rows of 64, four wavefronts per workgroup. The cross-tile part is `unsafe()` text, as
in the reference, and for this target that text is HIP: one 64-bit status word per tile (flag in the upper half,
value in the lower), written and polled with relaxed agent-scope atomics, so that a record is visible across the
XCDs' L2s in one piece; the look-back poll is bounded, so a broken ordering would show as a wrong result and
never as a hang.

CPU: the structure of the generated text (device functions before their callers, where the barriers land).
GPU: bit for bit against numpy's wrapping cumulative sum.
"""
import ctypes

import numpy as np
import pytest

from prism_amd import hipgen
from prism_amd.hipgen import (block, const, generate, generate_launcher, grid, group, partition, prism, ptr, requires,
                              shared, thread, uint32_t, uint64_t, unsafe)

TILE = 1024


@requires(thread[1])
@prism("device")
def shift_up_in_wavefront(val: uint32_t @ thread[1], delta: uint32_t @ thread[1]) -> uint32_t @ thread[1]:
    with group(thread[1]):
        unsafe("return __shfl_up(val, delta, 64);")
    return


@requires(grid[1])
@prism("device")
def take_ticket(counter: ptr(uint32_t) @ grid[1]) -> uint32_t @ grid[1]:
    """Tiles are numbered in the order in which workgroups start, so a tile only waits for tiles that run."""
    unsafe("""
__shared__ uint32_t ticket;
if (threadIdx.x == 0) ticket = atomicAdd(counter, 1u);
__syncthreads();
return ticket;
""")
    return


@requires(block[1], thread[1])
@prism("device")
def publish(status: ptr(uint64_t) @ block[1], tile: uint32_t @ block[1], flag: uint32_t @ block[1], value: uint32_t @ block[1]):
    """flag 1: `value` is the tile's own sum; flag 2: the sum of everything up to and including the tile."""
    with group(block[1]):
        unsafe("""
if (threadIdx.x == 0)
    __hip_atomic_store(&status[tile], (static_cast<uint64_t>(flag) << 32) | value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
""")
    return


@requires(block[1], thread[1])
@prism("device")
def look_back(status: ptr(uint64_t) @ block[1], tile: uint32_t @ block[1], spin_limit: int @ block[1]) -> uint32_t @ block[1]:
    """Sum of all tiles before `tile`: walks back over the published sums until it meets an inclusive prefix."""
    with group(block[1]):
        unsafe("""
__shared__ uint32_t before;
if (threadIdx.x == 0) {
    uint32_t sum = 0;
    for (int id = static_cast<int>(tile) - 1; id >= 0; --id) {
        uint64_t word = 0;
        for (int spins = 0; spins < spin_limit; ++spins) {
            word = __hip_atomic_load(&status[id], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (word >> 32) break;
            __builtin_amdgcn_s_sleep(1);
        }
        sum += static_cast<uint32_t>(word);
        if ((word >> 32) != 1) break;  // an inclusive prefix ends the walk (and so does a poll that ran out)
    }
    before = sum;
}
__syncthreads();
return before;
""")
    return


@requires(grid[1], block[1], thread[64])
@prism("global")
def lookback_scan(x: ptr(const(uint32_t)) @ grid[1], y: ptr(uint32_t) @ grid[1], counter: ptr(uint32_t) @ grid[1],
                  status: ptr(uint64_t) @ grid[1], spin_limit: int @ grid[1]):
    tile: uint32_t @ grid[1] = take_ticket(counter)
    with partition(x, p=block[1], offset=tile * 1024) as x_tile:
        with partition(y, p=block[1], offset=tile * 1024) as y_tile:
            with group(block[1]):
                scanned: shared(uint32_t[1024], static=True) @ block[1]
                ends: shared(uint32_t[16], static=True) @ block[1]
                upto: shared(uint32_t[16], static=True) @ block[1]
                wave: int @ thread[64] = id()
                # every wavefront scans four rows of 64 with lane shifts
                for i in range(4):
                    with partition(x_tile, p=thread[64], offset=(wave + 4 * i) * 64) as x_row:
                        with partition(scanned, p=thread[64], offset=(wave + 4 * i) * 64) as s_row:
                            with group(thread[64]):
                                lane: uint32_t @ thread[1] = id()
                                with group(thread[1]):
                                    v: uint32_t @ thread[1] = x_row[lane]
                                    stride: uint32_t @ thread[1] = 1
                                    while stride < 64:
                                        got: uint32_t @ thread[1] = shift_up_in_wavefront(v, stride)
                                        if lane >= stride:
                                            v = got + v
                                        stride *= 2
                                    s_row[lane] = v
                                    if lane == 63:
                                        ends[wave + 4 * i] = v
                # the first wavefront scans the sixteen row ends
                with group(thread[64]):
                    lane16: uint32_t @ thread[1] = id()
                    with group(thread[1]):
                        if wave == 0:
                            e: uint32_t @ thread[1] = 0
                            if lane16 < 16:
                                e = ends[lane16]
                            step: uint32_t @ thread[1] = 1
                            while step < 16:
                                below: uint32_t @ thread[1] = shift_up_in_wavefront(e, step)
                                if lane16 >= step:
                                    e = below + e
                                step *= 2
                            if lane16 < 16:
                                upto[lane16] = e
                total: uint32_t @ block[1] = upto[15]
                publish(status, tile, 1, total)
                before: uint32_t @ block[1] = look_back(status, tile, spin_limit)
                publish(status, tile, 2, before + total)
                t: int @ thread[1] = id()
                with group(thread[1]):
                    for k in range(4):
                        el: int @ thread[1] = t + 256 * k
                        row: int @ thread[1] = el / 64
                        base: uint32_t @ thread[1] = before
                        if row > 0:
                            base = before + upto[row - 1]
                        y_tile[el] = base + scanned[el]


def lines(text):
    return [ln.strip() for ln in text.splitlines()]


def test_structure_of_the_generated_scan():
    got = lines(generate("lookback_scan"))
    assert got[0] == ("__global__ void lookback_scan(const uint32_t* x, uint32_t* y, uint32_t* counter, uint64_t* status, "
                      "int spin_limit) {")
    assert "uint32_t tile = take_ticket(__block_id_0, __thread_id_0, __smem, counter);" in got
    assert "__shared__ uint32_t scanned[1024];" in got and "__shared__ uint32_t upto[16];" in got
    assert "int wave = (__thread_id_1 / 64);" in got
    assert "publish(__block_id_1, __thread_id_1, __smem, status, tile, 2, (before + total));" in got
    # barriers: in front of the `if` in which the first wavefront reads the row ends, in front of the read of the
    # total, and none inside a branch; the write-back reads arrays that are complete by then
    sync = [n for n, ln in enumerate(got) if ln == "__syncthreads();"]
    assert len(sync) == 2
    assert got[sync[0] + 1] == "if ((wave == 0)) {" and got[sync[1] + 1] == "uint32_t total = upto[15];"
    launcher = generate_launcher("lookback_scan")
    kernel_at = launcher.index(" lookback_scan(")
    assert all(launcher.index(f" {name}(") < kernel_at for name in ("shift_up_in_wavefront", "take_ticket", "publish", "look_back"))
    assert "__hip_atomic_store(&status[tile]" in launcher and "__shfl_up(val, delta, 64)" in launcher


@pytest.fixture(scope="module")
def built(tmp_path_factory):
    return hipgen.build("lookback_scan", out_dir=str(tmp_path_factory.mktemp("hipgen_scan")), block_size=256)


def test_launcher_compiles_for_gfx950(built):
    assert hasattr(built, "lookback_scan_launch")


@pytest.mark.gpu
@pytest.mark.parametrize("tiles", [1, 2, 7, 300, 4096])
def test_generated_lookback_scan_is_bit_exact(built, tiles):
    import torch
    fn = built.lookback_scan_launch
    fn.argtypes = [ctypes.c_void_p] * 4 + [ctypes.c_int, ctypes.c_uint, ctypes.c_void_p]
    n = tiles * TILE
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
