"""add_m: y = x + m, at block / thread level and by whole wavefronts.

`add_m_blocks` is the block-and-thread form of the reference's first example (examples/add_m_block_thread.py),
with a guard so that any element count is legal. `add_m_by_wavefronts` moves its data with the four load / store
building blocks of examples/thread_load.py, thread_store.py, warp_load.py:13-22 and warp_store.py, here on 64 lanes:
`lane_load` / `lane_store` copy a thread's own run of items, `wave_load` / `wave_store` give lane l of a wavefront
the l-th run (the blocked arrangement).
"""
from prism_amd.hipgen import block, const, grid, group, partition, prism, ptr, requires, thread


@requires(grid[1], block[1], thread[1])
@prism("global")
def add_m_blocks(x: ptr(const(int)) @ grid[1], y: ptr(int) @ grid[1], m: int @ grid[1],
                 per_block: int @ grid[1], n: int @ grid[1]):
    first: int @ block[1] = id() * per_block
    with partition(x, p=block[1], offset=first) as x_blk:
        with partition(y, p=block[1], offset=first) as y_blk:
            with group(block[1]):
                lane: int @ thread[1] = id()
                with partition(x_blk, p=thread[1], offset=lane) as x_one:
                    with partition(y_blk, p=thread[1], offset=lane) as y_one:
                        with group(thread[1]):
                            if first + lane < n:
                                y_one[0] = x_one[0] + m


@requires(thread[1])
@prism("device")
def lane_load(src: ptr(const(int)) @ thread[1], dst: ptr(int) @ thread[1], items: int @ thread[1]):
    with group(thread[1]):
        for i in range(items):
            dst[i] = src[i]


@requires(thread[1])
@prism("device")
def lane_store(src: ptr(const(int)) @ thread[1], dst: ptr(int) @ thread[1], items: int @ thread[1]):
    with group(thread[1]):
        for i in range(items):
            dst[i] = src[i]


@requires(thread[64])
@prism("device")
def wave_load(src: ptr(const(int)) @ thread[64], dst: ptr(int) @ thread[1], items: int @ thread[64]):
    """Blocked arrangement: lane l of the wavefront takes items l * items .. l * items + items - 1 of the
    wavefront's range (the reference's warp_load, examples/warp_load.py:13-22, on 64 lanes)."""
    with group(thread[64]):
        lane: int @ thread[1] = id()
        with partition(src, p=thread[1], offset=lane * items) as mine:
            with group(thread[1]):
                lane_load(mine, dst, items)


@requires(thread[64])
@prism("device")
def wave_store(src: ptr(const(int)) @ thread[1], dst: ptr(int) @ thread[64], items: int @ thread[64]):
    with group(thread[64]):
        lane: int @ thread[1] = id()
        with partition(dst, p=thread[1], offset=lane * items) as mine:
            with group(thread[1]):
                lane_store(src, mine, items)


@requires(grid[1], block[1], thread[64])
@prism("global")
def add_m_by_wavefronts(x: ptr(const(int)) @ grid[1], y: ptr(int) @ grid[1], m: int @ grid[1], wavefronts: int @ grid[1]):
    """Every wavefront loads 64 x 4 consecutive elements into registers, adds m and stores them."""
    w: int @ thread[64] = id()
    with partition(x, p=thread[64], offset=w * 256) as x_wave:
        with partition(y, p=thread[64], offset=w * 256) as y_wave:
            with group(block[1]):
                with group(thread[64]):
                    held: int[4] @ thread[1]
                    if w < wavefronts:
                        wave_load(x_wave, held, 4)
                        for i in range(4):
                            held[i] += m
                        wave_store(held, y_wave, 4)
