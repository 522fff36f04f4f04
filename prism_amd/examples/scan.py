"""Prefix sums: a row scan by lane shifts and a single-pass scan with decoupled look-back, twice.

The look-back scan follows the decomposition of the reference's example (examples/scan.py: a ticket from a global
counter :88-99, row scans by lane shifts :106-128, the scan of the row ends :147-173, aggregate / prefix records and
the look-back in target text :34-85, the write-back with the tile's prefix :176-193) on 64-lane wavefronts: a tile
is 1024 elements = 16 rows of 64, four wavefronts per workgroup. `lookback_scan` is one kernel body;
`lookback_scan_by_parts` is the same scan as a chain of device functions that are handed the LDS arrays, the way
the reference's kernel is put together (examples/scan.py:195-224). The cross-tile part is `unsafe()` text, as in the
reference, and for this target that text is HIP: one 64-bit status word per tile (flag in the upper half, value in
the lower), written and polled with relaxed agent-scope atomics, so that a record is visible across the XCDs' L2s
in one piece; the look-back poll is bounded, so a broken ordering would show as a wrong result and never as a hang.
"""
from prism_amd.hipgen import block, const, grid, group, partition, prism, ptr, requires, shared, thread, uint32_t, uint64_t, unsafe


@requires(thread[1])
@prism("device")
def lane_shift_up(val: uint32_t @ thread[1], delta: uint32_t @ thread[1]) -> uint32_t @ thread[1]:
    with group(thread[1]):
        unsafe("return __shfl_up(val, delta, 32);")
    return


@requires(grid[1], block[1], thread[32])
@prism("global")
def row_scan32(x: ptr(const(uint32_t)) @ grid[1], y: ptr(uint32_t) @ grid[1], rows: int @ grid[1]):
    """Inclusive scan of every row of 32 elements by a group of 32 threads (half a wavefront), the
    building block of the reference's scan (scan_warps, examples/scan.py:106-128)."""
    first_row: int @ block[1] = id() * 8
    with partition(x, p=block[1], offset=first_row * 32) as x_blk:
        with partition(y, p=block[1], offset=first_row * 32) as y_blk:
            with group(block[1]):
                g: int @ thread[32] = id()
                with partition(x_blk, p=thread[32], offset=g * 32) as x_row:
                    with partition(y_blk, p=thread[32], offset=g * 32) as y_row:
                        with group(thread[32]):
                            lane: uint32_t @ thread[1] = id()
                            with partition(y_row, p=thread[1], offset=lane) as y_one:
                                with group(thread[1]):
                                    v: uint32_t @ thread[1] = 0
                                    if first_row + g < rows:
                                        v = x_row[lane]
                                    step: uint32_t @ thread[1] = 1
                                    while step < 32:
                                        got: uint32_t @ thread[1] = lane_shift_up(v, step)
                                        if lane >= step:
                                            v = got + v
                                        step *= 2
                                    if first_row + g < rows:
                                        y_one[0] = v


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
            with partition(status, p=block[1], offset=0) as status_blk:
                with group(block[1]):
                    scanned: shared(uint32_t[1024], static=True) @ block[1]
                    ends: shared(uint32_t[16], static=True) @ block[1]
                    upto: shared(uint32_t[16], static=True) @ block[1]
                    wave: int @ thread[64] = id()
                    # every wavefront scans four rows of 64 with lane shifts
                    for i in range(4):
                        with partition(x_tile, p=thread[64], offset=(wave + 4 * i) * 64) as x_row:
                            with partition(scanned, p=thread[64], offset=(wave + 4 * i) * 64) as s_row:
                                with partition(ends, p=thread[64], offset=wave + 4 * i) as row_end:
                                    with group(thread[64]):
                                        lane: uint32_t @ thread[1] = id()
                                        with partition(s_row, p=thread[1], offset=lane) as s_one:
                                            with partition(row_end, p=thread[1], offset=0) as end_one:
                                                with group(thread[1]):
                                                    v: uint32_t @ thread[1] = x_row[lane]
                                                    stride: uint32_t @ thread[1] = 1
                                                    while stride < 64:
                                                        got: uint32_t @ thread[1] = shift_up_in_wavefront(v, stride)
                                                        if lane >= stride:
                                                            v = got + v
                                                        stride *= 2
                                                    s_one[0] = v
                                                    if lane == 63:
                                                        end_one[0] = v
                    # the first wavefront scans the sixteen row ends
                    with partition(upto, p=thread[64], offset=0) as upto_wave:
                        with group(thread[64]):
                            lane16: uint32_t @ thread[1] = id()
                            with partition(upto_wave, p=thread[1], offset=lane16) as upto_one:
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
                                            upto_one[0] = e
                    total: uint32_t @ block[1] = upto[15]
                    publish(status_blk, tile, 1, total)
                    before: uint32_t @ block[1] = look_back(status_blk, tile, spin_limit)
                    publish(status_blk, tile, 2, before + total)
                    t: int @ thread[1] = id()
                    with partition(y_tile, p=thread[1], offset=t) as y_mine:
                        with group(thread[1]):
                            for k in range(4):
                                el: int @ thread[1] = t + 256 * k
                                row: int @ thread[1] = el / 64
                                base: uint32_t @ thread[1] = before
                                if row > 0:
                                    base = before + upto[row - 1]
                                y_mine[256 * k] = base + scanned[el]


@requires(block[1], thread[64])
@prism("device")
def scan_rows(x_tile: ptr(const(uint32_t)) @ block[1], scanned: ptr(shared(uint32_t)) @ block[1]):
    """Every wavefront scans four rows of 64 elements with lane shifts and stores them."""
    with group(block[1]):
        wave: int @ thread[64] = id()
        for i in range(4):
            with partition(x_tile, p=thread[64], offset=(wave + 4 * i) * 64) as x_row:
                with partition(scanned, p=thread[64], offset=(wave + 4 * i) * 64) as s_row:
                    with group(thread[64]):
                        lane: uint32_t @ thread[1] = id()
                        with partition(s_row, p=thread[1], offset=lane) as s_one:
                            with group(thread[1]):
                                v: uint32_t @ thread[1] = x_row[lane]
                                stride: uint32_t @ thread[1] = 1
                                while stride < 64:
                                    got: uint32_t @ thread[1] = shift_up_in_wavefront(v, stride)
                                    if lane >= stride:
                                        v = got + v
                                    stride *= 2
                                s_one[0] = v
    return


@requires(block[1], thread[64])
@prism("device")
def collect_row_ends(scanned: ptr(const(shared(uint32_t))) @ block[1], ends: ptr(shared(uint32_t)) @ block[1]):
    with group(block[1]):
        t: uint32_t @ thread[1] = id()
        with partition(ends, p=thread[1], offset=t) as end_one:
            with group(thread[1]):
                if t < 16:
                    end_one[0] = scanned[64 * t + 63]
    return


@requires(block[1], thread[64])
@prism("device")
def scan_row_ends(ends: ptr(shared(uint32_t)) @ block[1], spare: ptr(shared(uint32_t)) @ block[1]) -> ptr(uint32_t) @ block[1]:
    """Sixteen sums scanned in four doubling steps through a second array; returns where the result is, which
    is complete for every thread when the function returns."""
    with group(block[1]):
        t: uint32_t @ thread[1] = id()
        stride: uint32_t @ block[1] = 1
        while stride < 16:
            with partition(ends, p=thread[1], offset=t) as end_one:
                with partition(spare, p=thread[1], offset=t) as spare_one:
                    with group(thread[1]):
                        if t < 16:
                            if t >= stride:
                                spare_one[0] = ends[t] + ends[t - stride]
                            else:
                                spare_one[0] = ends[t]
                        if t < 16:
                            end_one[0] = spare[t]
            stride *= 2
    return ends


@requires(block[1], thread[64])
@prism("device")
def write_back(y_tile: ptr(uint32_t) @ block[1], scanned: ptr(const(shared(uint32_t))) @ block[1],
               upto: ptr(const(uint32_t)) @ block[1], before: uint32_t @ block[1]):
    with group(block[1]):
        t: int @ thread[1] = id()
        with partition(y_tile, p=thread[1], offset=t) as y_mine:
            with group(thread[1]):
                for k in range(4):
                    el: int @ thread[1] = t + 256 * k
                    row: int @ thread[1] = el / 64
                    base: uint32_t @ thread[1] = before
                    if row > 0:
                        base = before + upto[row - 1]
                    y_mine[256 * k] = base + scanned[el]
    return


@requires(grid[1], block[1], thread[64])
@prism("global")
def lookback_scan_by_parts(x: ptr(const(uint32_t)) @ grid[1], y: ptr(uint32_t) @ grid[1], counter: ptr(uint32_t) @ grid[1],
                           status: ptr(uint64_t) @ grid[1], spin_limit: int @ grid[1]):
    tile: uint32_t @ grid[1] = take_ticket(counter)
    with partition(x, p=block[1], offset=tile * 1024) as x_tile:
        with partition(y, p=block[1], offset=tile * 1024) as y_tile:
            with partition(status, p=block[1], offset=0) as status_blk:
                with group(block[1]):
                    scanned: shared(uint32_t[1024], static=True) @ block[1]
                    scan_rows(x_tile, scanned)
                    ends: shared(uint32_t[16], static=True) @ block[1]
                    spare: shared(uint32_t[16], static=True) @ block[1]
                    collect_row_ends(scanned, ends)
                    upto: ptr(uint32_t) @ block[1] = scan_row_ends(ends, spare)
                    total: uint32_t @ block[1] = upto[15]
                    publish(status_blk, tile, 1, total)
                    before: uint32_t @ block[1] = look_back(status_blk, tile, spin_limit)
                    publish(status_blk, tile, 2, before + total)
                    write_back(y_tile, scanned, upto, before)


# The look-back scan with sixteen elements per thread and a look-back that reads 64 status words at a time.

@requires(block[1], thread[1])
@prism("device")
def look_back_wide(status: ptr(uint64_t) @ block[1], tile: uint32_t @ block[1], spin_limit: int @ block[1]) -> uint32_t @ block[1]:
    """Sum of all tiles before `tile`. The first wavefront reads the status words of the 64 tiles before it at once
    (lane 0 the nearest), waits until every word between this tile and the nearest inclusive prefix is there, adds
    them up, and moves on by 64 tiles if the window held no prefix. Tiles before the first count as a prefix of 0.
    The wait is bounded: a broken ordering shows as a wrong result, never as a hang."""
    with group(block[1]):
        unsafe("""
__shared__ uint32_t before;
if (threadIdx.x < 64) {
    uint32_t sum = 0;
    int nearest = static_cast<int>(tile) - 1, spins = 0;
    bool done = false;
    while (!done) {
        const int id = nearest - static_cast<int>(threadIdx.x);
        for (;;) {
            const uint64_t word = id >= 0 ? __hip_atomic_load(&status[id], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                                          : (static_cast<uint64_t>(2) << 32);
            const uint64_t prefixes = __ballot((word >> 32) == 2), missing = __ballot((word >> 32) == 0);
            const int first = prefixes ? __ffsll(static_cast<unsigned long long>(prefixes)) - 1 : 64;
            const uint64_t wanted = first >= 63 ? ~0ull : ((1ull << (first + 1)) - 1);
            if ((missing & wanted) == 0 || ++spins > spin_limit) {
                uint32_t part = static_cast<int>(threadIdx.x) <= first ? static_cast<uint32_t>(word) : 0u;
                for (int o = 32; o > 0; o >>= 1) part += __shfl_xor(part, o, 64);
                sum += part;
                done = first < 64 || spins > spin_limit;
                nearest -= 64;
                break;
            }
            __builtin_amdgcn_s_sleep(1);
        }
    }
    if (threadIdx.x == 0) before = sum;
}
__syncthreads();
return before;
""")
    return


@requires(grid[1], block[1], thread[64])
@prism("global")
def lookback_scan_wide(x: ptr(const(uint32_t)) @ grid[1], y: ptr(uint32_t) @ grid[1], counter: ptr(uint32_t) @ grid[1],
                       status: ptr(uint64_t) @ grid[1], spin_limit: int @ grid[1]):
    """Tiles of 4096 elements, 256 threads with 16 consecutive elements each in a private array: a serial scan per
    thread, one scan by lane shifts over the thread totals of a wavefront, the four wavefront totals through LDS."""
    tile: uint32_t @ grid[1] = take_ticket(counter)
    with partition(x, p=block[1], offset=tile * 4096) as x_tile:
        with partition(y, p=block[1], offset=tile * 4096) as y_tile:
            with partition(status, p=block[1], offset=0) as status_blk:
                with group(block[1]):
                    wave_sums: shared(uint32_t[4], static=True) @ block[1]
                    t: int @ thread[1] = id()
                    wave: int @ thread[64] = id()
                    v: uint32_t[16] @ thread[1]
                    with partition(x_tile, p=thread[1], offset=16 * t) as x_mine:
                        with group(thread[1]):
                            for i in range(16):
                                v[i] = x_mine[i]
                            for i in range(1, 16):
                                v[i] += v[i - 1]
                    upto_me: uint32_t @ thread[1] = v[15]
                    with partition(wave_sums, p=thread[64], offset=wave) as my_wave_sum:
                        with group(thread[64]):
                            lane: uint32_t @ thread[1] = id()
                            with partition(my_wave_sum, p=thread[1], offset=0) as sum_one:
                                with group(thread[1]):
                                    stride: uint32_t @ thread[1] = 1
                                    while stride < 64:
                                        got: uint32_t @ thread[1] = shift_up_in_wavefront(upto_me, stride)
                                        if lane >= stride:
                                            upto_me = got + upto_me
                                        stride *= 2
                                    if lane == 63:
                                        sum_one[0] = upto_me
                    total: uint32_t @ block[1] = wave_sums[0] + wave_sums[1] + wave_sums[2] + wave_sums[3]
                    publish(status_blk, tile, 1, total)
                    before: uint32_t @ block[1] = look_back_wide(status_blk, tile, spin_limit)
                    publish(status_blk, tile, 2, before + total)
                    with partition(y_tile, p=thread[1], offset=16 * t) as y_mine:
                        with group(thread[64]):
                            earlier_waves: uint32_t @ thread[64] = 0
                            for w in range(4):
                                if w < wave:
                                    earlier_waves += wave_sums[w]
                            with group(thread[1]):
                                base: uint32_t @ thread[1] = before + earlier_waves + (upto_me - v[15])
                                for i in range(16):
                                    y_mine[i] = base + v[i]


# The same scan with the tile read the way the memory system likes it: a lane's 16 bytes next to its neighbour's.

@requires(thread[1])
@prism("device")
def value_of_last_lane(val: uint32_t @ thread[1]) -> uint32_t @ thread[1]:
    with group(thread[1]):
        unsafe("return __shfl(val, 63, 64);")
    return


@requires(grid[1], block[1], thread[64])
@prism("global")
def lookback_scan_striped(x: ptr(const(uint32_t)) @ grid[1], y: ptr(uint32_t) @ grid[1], counter: ptr(uint32_t) @ grid[1],
                          status: ptr(uint64_t) @ grid[1], spin_limit: int @ grid[1]):
    """Tiles of 65536 elements as 256 rows of 256 (1024 threads); a wavefront owns sixteen consecutive rows and a lane
    four consecutive elements of each (one 16-byte access per row, the 64 lanes of an access side by side). Per row: the lane's
    four elements serially, the lane totals by lane shifts, and what the wavefront's earlier rows hold added on."""
    tile: uint32_t @ grid[1] = take_ticket(counter)
    with partition(x, p=block[1], offset=tile * 65536) as x_tile:
        with partition(y, p=block[1], offset=tile * 65536) as y_tile:
            with partition(status, p=block[1], offset=0) as status_blk:
                with group(block[1]):
                    wave_sums: shared(uint32_t[16], static=True) @ block[1]
                    wave: int @ thread[64] = id()
                    v: uint32_t[64] @ thread[1]
                    with partition(x_tile, p=thread[64], offset=4096 * wave) as x_wave:
                        with partition(wave_sums, p=thread[64], offset=wave) as my_wave_sum:
                            with group(thread[64]):
                                lane: uint32_t @ thread[1] = id()
                                with partition(x_wave, p=thread[1], offset=4 * lane) as x_mine:
                                    with partition(my_wave_sum, p=thread[1], offset=0) as sum_one:
                                        with group(thread[1]):
                                            for j in range(16):
                                                for e in range(4):
                                                    v[4 * j + e] = x_mine[256 * j + e]
                                            carry: uint32_t @ thread[1] = 0
                                            for j in range(16):
                                                v[4 * j + 1] += v[4 * j]
                                                v[4 * j + 2] += v[4 * j + 1]
                                                v[4 * j + 3] += v[4 * j + 2]
                                                upto_me: uint32_t @ thread[1] = v[4 * j + 3]
                                                stride: uint32_t @ thread[1] = 1
                                                while stride < 64:
                                                    got: uint32_t @ thread[1] = shift_up_in_wavefront(upto_me, stride)
                                                    if lane >= stride:
                                                        upto_me = got + upto_me
                                                    stride *= 2
                                                ahead: uint32_t @ thread[1] = carry + (upto_me - v[4 * j + 3])
                                                for e in range(4):
                                                    v[4 * j + e] += ahead
                                                carry += value_of_last_lane(upto_me)
                                            if lane == 63:
                                                sum_one[0] = carry
                    total: uint32_t @ block[1] = 0
                    for w in range(16):
                        total += wave_sums[w]
                    publish(status_blk, tile, 1, total)
                    before: uint32_t @ block[1] = look_back_wide(status_blk, tile, spin_limit)
                    publish(status_blk, tile, 2, before + total)
                    with partition(y_tile, p=thread[64], offset=4096 * wave) as y_wave:
                        with group(thread[64]):
                            lane_out: uint32_t @ thread[1] = id()
                            earlier_waves: uint32_t @ thread[64] = 0
                            for w in range(16):
                                if w < wave:
                                    earlier_waves += wave_sums[w]
                            with partition(y_wave, p=thread[1], offset=4 * lane_out) as y_mine:
                                with group(thread[1]):
                                    for j in range(16):
                                        for e in range(4):
                                            y_mine[256 * j + e] = before + earlier_waves + v[4 * j + e]
