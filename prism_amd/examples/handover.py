"""A producer wavefront and four consumer wavefronts in one workgroup: D = P Q^T in bf16 with fp32 sums.

The shape of the reference's H100 kernel (examples/h100_matmul.py:120-258): `match split(thread)` gives the first
members of the workgroup the loads and the rest the matrix instructions, the tiles travel through LDS slots that the
producer claims, and nobody writes a barrier: the generator sees that one case writes a slot and another reads it
and hands the slot back and forth. What the reference does with tensor-map loads, mbarriers and wgmma is done here
with what gfx950 has: loads that go from global memory straight into LDS (64 lanes x 16 bytes per instruction, so a
tile row of 32 bf16 is four lanes wide and one instruction fills 16 rows), two round counters per slot in LDS, and
the 16x16x32 bf16 matrix instruction fed by 16-byte LDS reads.

A workgroup owns a 64 x 64 tile of D. P is M x K and Q is N x K, both with K contiguous; per step of 64 along K the
producer fills two pairs of slots (32 k each) and each consumer wavefront multiplies its 16 rows of the P slot with
the four 16-row groups of the Q slot. While the consumers work on one pair of slots the producer fills the other.
M and N are multiples of 64, K of 64.
"""
from prism_amd.hipgen import attr, bf16, block, claim, const, float4, float4_cast, grid, group, intrinsic, partition, prism, ptr, requires, shared, split, thread


@requires(grid[1], block[1], thread[320])
@prism("global")
def handed_over_gemm(P: ptr(const(bf16)) @ grid[1], Q: ptr(const(bf16)) @ grid[1], D: ptr(float) @ grid[1],
                     N: int @ grid[1], K: int @ grid[1], tiles_n: int @ grid[1]):
    tile_r: const(int) @ block[1] = id() / tiles_n
    tile_c: const(int) @ block[1] = id() % tiles_n
    with partition(P, p=block[1], offset=tile_r * 64 * K) as P_rows:
        with partition(Q, p=block[1], offset=tile_c * 64 * K) as Q_rows:
            with partition(D, p=block[1], offset=tile_r * 64 * N + tile_c * 64) as D_tile:
                with group(block[1]):
                    p_first: shared(bf16[2048], static=True) @ block[1]     # 64 rows x 32 k
                    q_first: shared(bf16[2048], static=True) @ block[1]
                    p_second: shared(bf16[2048], static=True) @ block[1]
                    q_second: shared(bf16[2048], static=True) @ block[1]
                    acc: float[16] @ thread[1] = {0}
                    for k0 in range(0, K, 64):
                        with claim(p_first, p=thread[64], offset=0) as p_first_fill:
                            with claim(q_first, p=thread[64], offset=0) as q_first_fill:
                                with claim(p_second, p=thread[64], offset=0) as p_second_fill:
                                    with claim(q_second, p=thread[64], offset=0) as q_second_fill:
                                        match split(thread):
                                            case 64:
                                                with group(thread[64]):
                                                    lane: int @ thread[1] = id()
                                                    row: int @ thread[1] = lane / 4
                                                    k8: int @ thread[1] = 8 * (lane % 4)
                                                    for part in range(4):
                                                        intrinsic.load_to_lds(p_first_fill[512 * part],
                                                                              P_rows[(16 * part + row) * K + k0 + k8])
                                                        intrinsic.load_to_lds(q_first_fill[512 * part],
                                                                              Q_rows[(16 * part + row) * K + k0 + k8])
                                                    for part in range(4):
                                                        intrinsic.load_to_lds(p_second_fill[512 * part],
                                                                              P_rows[(16 * part + row) * K + k0 + 32 + k8])
                                                        intrinsic.load_to_lds(q_second_fill[512 * part],
                                                                              Q_rows[(16 * part + row) * K + k0 + 32 + k8])
                                            case 256:
                                                wave: int @ thread[64] = id()
                                                with group(thread[64]):
                                                    lane: int @ thread[1] = id()
                                                    r: int @ thread[1] = lane % 16
                                                    k8: int @ thread[1] = 8 * (lane / 16)
                                                    a: float4 @ thread[1] = float4_cast(p_first[(16 * wave + r) * 32 + k8])
                                                    for n in range(4):
                                                        b: float4 @ thread[1] = float4_cast(q_first[(16 * n + r) * 32 + k8])
                                                        intrinsic.mfma_f32_16x16x32_bf16(
                                                            a, b, acc[4 * n], acc[4 * n + 1], acc[4 * n + 2], acc[4 * n + 3],
                                                            out=[acc[4 * n], acc[4 * n + 1], acc[4 * n + 2], acc[4 * n + 3]])
                                                    a2: float4 @ thread[1] = float4_cast(p_second[(16 * wave + r) * 32 + k8])
                                                    for n in range(4):
                                                        b2: float4 @ thread[1] = float4_cast(q_second[(16 * n + r) * 32 + k8])
                                                        intrinsic.mfma_f32_16x16x32_bf16(
                                                            a2, b2, acc[4 * n], acc[4 * n + 1], acc[4 * n + 2], acc[4 * n + 3],
                                                            out=[acc[4 * n], acc[4 * n + 1], acc[4 * n + 2], acc[4 * n + 3]])
                    with partition(D_tile, p=thread[1], offset=0) as D_mine:
                        match split(thread):
                            case 64:
                                pass
                            case 256:
                                wave: int @ thread[64] = id()
                                with group(thread[64]):
                                    lane: int @ thread[1] = id()
                                    with group(thread[1]):
                                        for n in range(4):
                                            for v in range(4):
                                                D_mine[(16 * wave + 4 * (lane / 16) + v) * N + 16 * n + lane % 16] = acc[4 * n + v]


# The same hand-over at full size: a 128 x 256 tile per workgroup, four producer and four consumer wavefronts,
# three slots of 64 k (48 KiB each: 128 rows of P, then 256 rows of Q, 128-byte rows). The producers fill the
# slots in turn; because one case fills several arrays, the generator announces a filling only when the next
# one's loads are on their way, so that two fillings are in flight while the consumers multiply the third.
# Measured at 8192^3: eight consumers of 64 x 64 and two slots 1000 TFLOP/s, four of 64 x 128 and two slots
# 1030, four of 64 x 128 and three slots 1120.

@requires(thread[256])
@prism("device")
def fill_slot(slot: ptr(bf16) @ thread[256], P_from: ptr(const(bf16)) @ block[1], Q_from: ptr(const(bf16)) @ block[1],
              K: int @ grid[1], k_at: int @ block[1]):
    """Four wavefronts copy 128 rows x 64 k of P and 256 rows x 64 k of Q, starting at column k_at, into a slot.
    One direct load covers 8 rows. The 16-byte chunk c of row r is kept at position c ^ ((r / 2) % 8) of the row,
    so that the sixteen rows a quarter of a wavefront reads later fall into different LDS banks: a lane fetches
    the chunk that belongs where its 16 bytes land."""
    with group(thread[256]):
        w: int @ thread[64] = id()
        with group(thread[64]):
            lane: int @ thread[1] = id()
            for part in range(4):
                prow: int @ thread[1] = 8 * (4 * part + w) + lane / 8
                intrinsic.load_to_lds(slot[512 * (4 * part + w)],
                                      P_from[prow * K + k_at + 8 * ((lane % 8) ^ ((prow / 2) % 8))])
            for part in range(8):
                qrow: int @ thread[1] = 8 * (4 * part + w) + lane / 8
                intrinsic.load_to_lds(slot[8192 + 512 * (4 * part + w)],
                                      Q_from[qrow * K + k_at + 8 * ((lane % 8) ^ ((qrow / 2) % 8))])
    return


@requires(thread[256])
@prism("device")
def multiply_slot(acc: ptr(float) @ thread[1], slot: ptr(const(bf16)) @ block[1]):
    """Four wavefronts, two down and two across, each adding its 64 x 128 part of (P part)(Q part)^T to acc: two
    k-steps of 4 x 8 matrix instructions of 16 x 16 x 32, acc[(8 i + j) * 4 + v] = D[16 i + 4 (lane / 16) + v][16 j + lane % 16]."""
    with group(thread[256]):
        wave: int @ thread[64] = id()
        row0: int @ thread[64] = 64 * (wave / 2)
        col0: int @ thread[64] = 128 * (wave % 2)
        with group(thread[64]):
            lane: int @ thread[1] = id()
            r: int @ thread[1] = lane % 16
            a: float4[4] @ thread[1]
            for kk in range(2):
                k8: int @ thread[1] = 8 * ((4 * kk + lane / 16) ^ ((r / 2) % 8))
                for i in range(4):
                    a[i] = float4_cast(slot[(row0 + 16 * i + r) * 64 + k8])
                for j in range(8):
                    b: float4 @ thread[1] = float4_cast(slot[8192 + (col0 + 16 * j + r) * 64 + k8])
                    for i in range(4):
                        intrinsic.mfma_f32_16x16x32_bf16(
                            a[i], b, acc[(8 * i + j) * 4], acc[(8 * i + j) * 4 + 1], acc[(8 * i + j) * 4 + 2], acc[(8 * i + j) * 4 + 3],
                            out=[acc[(8 * i + j) * 4], acc[(8 * i + j) * 4 + 1], acc[(8 * i + j) * 4 + 2], acc[(8 * i + j) * 4 + 3]])
    return


@attr("__launch_bounds__(512)")
@requires(grid[1], block[1], thread[512])
@prism("global")
def handed_over_gemm_big(P: ptr(const(bf16)) @ grid[1], Q: ptr(const(bf16)) @ grid[1], D: ptr(float) @ grid[1],
                         N: int @ grid[1], K: int @ grid[1], tiles_m: int @ grid[1], tiles_n: int @ grid[1]):
    """D = P Q^T on 128 x 256 tiles: 256 producer threads keep three slots filled, 256 consumer threads multiply
    them. K is a multiple of 64, M of 1024 and N of 256 (tiles_m = M / 128 a multiple of 8, tiles_n = N / 256).
    Workgroups are dealt to the eight XCDs in turn; the tile order gives the workgroups that run on one XCD at the
    same time a patch of eight tile rows by four tile columns, so that they share their panels in its L2.
    A trip of the loop covers 192 k. Where K ends inside a trip the producers fill the remaining slots with the
    first K tiles once more (every trip issues the same loads, which is what lets the generator count them) and
    the consumers leave those slots out."""
    per_xcd: const(int) @ block[1] = (tiles_m * tiles_n) / 8
    t: const(int) @ block[1] = (id() % 8) * per_xcd + id() / 8
    tile_r: const(int) @ block[1] = 8 * (t / (8 * tiles_n)) + t % 8
    tile_c: const(int) @ block[1] = (t % (8 * tiles_n)) / 8
    with partition(P, p=block[1], offset=tile_r * 128 * K) as P_rows:
        with partition(Q, p=block[1], offset=tile_c * 256 * K) as Q_rows:
            with partition(D, p=block[1], offset=tile_r * 128 * N + tile_c * 256) as D_tile:
                with group(block[1]):
                    first: shared(bf16[24576], static=True) @ block[1]
                    second: shared(bf16[24576], static=True) @ block[1]
                    third: shared(bf16[24576], static=True) @ block[1]
                    acc: float[128] @ thread[1] = {0}
                    for k0 in range(0, K, 192):
                        k1: const(int) @ block[1] = (k0 + 64) % K
                        k2: const(int) @ block[1] = (k0 + 128) % K
                        with claim(first, p=thread[256], offset=0) as first_fill:
                            with claim(second, p=thread[256], offset=0) as second_fill:
                                with claim(third, p=thread[256], offset=0) as third_fill:
                                    match split(thread):
                                        case 256:
                                            fill_slot(first_fill, P_rows, Q_rows, K, k0)
                                            fill_slot(second_fill, P_rows, Q_rows, K, k1)
                                            fill_slot(third_fill, P_rows, Q_rows, K, k2)
                                        case 256:
                                            multiply_slot(acc, first)
                                            if k0 + 64 < K:
                                                multiply_slot(acc, second)
                                            if k0 + 128 < K:
                                                multiply_slot(acc, third)
                    with partition(D_tile, p=thread[1], offset=0) as D_mine:
                        match split(thread):
                            case 256:
                                pass
                            case 256:
                                wave: int @ thread[64] = id()
                                with group(thread[64]):
                                    lane: int @ thread[1] = id()
                                    with group(thread[1]):
                                        for i in range(4):
                                            for j in range(8):
                                                for v in range(4):
                                                    D_mine[(64 * (wave / 2) + 16 * i + 4 * (lane / 16) + v) * N
                                                           + 128 * (wave % 2) + 16 * j + lane % 16] = acc[(8 * i + j) * 4 + v]


# SGEMM the same way: C = alpha A B + beta C (row-major fp32) on the fp32 matrix instruction, 128 x 256 tiles,
# two slots of 32 k (48 KiB each: 128 rows of A with 128-byte rows, then 32 rows of B with 1 KiB rows).
# Measured at 8192^3: 129 TFLOP/s; 150 with the loads taken out (hand-over still running, results invalid), so the
# protocol and the consumers' schedule cost 5 % and the loads 13 %; four slots of 16 k, which let the producers
# run further ahead, gave 124, three slots of 32 k 129, 256 x 256 tiles (42 registers spilled) 129: it is not the
# lead. One, two, four, eight producer wavefronts: 107, 126, 129, 128; fills staged through registers: 104.

@requires(thread[256])
@prism("device")
def fill_slot_f32(slot: ptr(float) @ thread[256], A_from: ptr(const(float)) @ block[1], B_from: ptr(const(float)) @ block[1],
                  N: int @ grid[1], K: int @ grid[1], k_at: int @ block[1]):
    """Four wavefronts copy 128 rows x 32 k of A (8 rows per direct load, 16-byte chunks placed at
    c ^ ((row / 2) % 8) as in fill_slot) and 32 k-rows x 256 columns of B (one k-row per direct load)."""
    with group(thread[256]):
        w: int @ thread[64] = id()
        with group(thread[64]):
            lane: int @ thread[1] = id()
            for part in range(4):
                arow: int @ thread[1] = 8 * (4 * part + w) + lane / 8
                intrinsic.load_to_lds(slot[256 * (4 * part + w)],
                                      A_from[arow * K + k_at + 4 * ((lane % 8) ^ ((arow / 2) % 8))])
            for part in range(8):
                intrinsic.load_to_lds(slot[4096 + 256 * (4 * part + w)], B_from[(k_at + 4 * part + w) * N + 4 * lane])
    return


@requires(thread[512])
@prism("device")
def multiply_slot_f32(acc: ptr(float) @ thread[1], slot: ptr(const(float)) @ block[1]):
    """Eight wavefronts, two down and four across, each adding its 64 x 64 part of (A part)(B part) to acc: sixteen
    pairs of k values, 2 x 2 instructions of 32 x 32 x 2 per pair;
    acc[(2 i + j) * 16 + v] = C[32 i + 8 (v / 4) + 4 (lane / 32) + v % 4][32 j + lane % 32]."""
    with group(thread[512]):
        wave: int @ thread[64] = id()
        row0: int @ thread[64] = 64 * (wave / 4)
        col0: int @ thread[64] = 64 * (wave % 4)
        with group(thread[64]):
            lane: int @ thread[1] = id()
            l32: int @ thread[1] = lane % 32
            a: float[2] @ thread[1]
            b: float[2] @ thread[1]
            for kk in range(0, 32, 2):
                k: int @ thread[1] = kk + lane / 32
                for i in range(2):
                    a[i] = slot[(row0 + 32 * i + l32) * 32 + 4 * ((k / 4) ^ ((l32 / 2) % 8)) + k % 4]
                for j in range(2):
                    b[j] = slot[4096 + k * 256 + col0 + 32 * j + l32]
                for i in range(2):
                    for j in range(2):
                        intrinsic.mfma_f32_32x32x2_f32(a[i], b[j], acc[(2 * i + j) * 16 + 0], acc[(2 * i + j) * 16 + 1], acc[(2 * i + j) * 16 + 2], acc[(2 * i + j) * 16 + 3], acc[(2 * i + j) * 16 + 4], acc[(2 * i + j) * 16 + 5], acc[(2 * i + j) * 16 + 6], acc[(2 * i + j) * 16 + 7], acc[(2 * i + j) * 16 + 8], acc[(2 * i + j) * 16 + 9], acc[(2 * i + j) * 16 + 10], acc[(2 * i + j) * 16 + 11], acc[(2 * i + j) * 16 + 12], acc[(2 * i + j) * 16 + 13], acc[(2 * i + j) * 16 + 14], acc[(2 * i + j) * 16 + 15],
                                                       out=[acc[(2 * i + j) * 16 + 0], acc[(2 * i + j) * 16 + 1], acc[(2 * i + j) * 16 + 2], acc[(2 * i + j) * 16 + 3], acc[(2 * i + j) * 16 + 4], acc[(2 * i + j) * 16 + 5], acc[(2 * i + j) * 16 + 6], acc[(2 * i + j) * 16 + 7], acc[(2 * i + j) * 16 + 8], acc[(2 * i + j) * 16 + 9], acc[(2 * i + j) * 16 + 10], acc[(2 * i + j) * 16 + 11], acc[(2 * i + j) * 16 + 12], acc[(2 * i + j) * 16 + 13], acc[(2 * i + j) * 16 + 14], acc[(2 * i + j) * 16 + 15]])
    return


@attr("__launch_bounds__(768)")
@requires(grid[1], block[1], thread[768])
@prism("global")
def handed_over_sgemm(M: int @ grid[1], N: int @ grid[1], K: int @ grid[1], alpha: float @ grid[1],
                      A: ptr(const(float)) @ grid[1], B: ptr(const(float)) @ grid[1], beta: float @ grid[1],
                      C: ptr(float) @ grid[1], tiles_n: int @ grid[1]):
    """M a multiple of 1024, N of 256, K of 64; tiles_n = N / 256. Tile order as in handed_over_gemm_big."""
    per_xcd: const(int) @ block[1] = ((M / 128) * tiles_n) / 8
    t: const(int) @ block[1] = (id() % 8) * per_xcd + id() / 8
    tile_r: const(int) @ block[1] = 8 * (t / (8 * tiles_n)) + t % 8
    tile_c: const(int) @ block[1] = (t % (8 * tiles_n)) / 8
    with partition(A, p=block[1], offset=tile_r * 128 * K) as A_rows:
        with partition(B, p=block[1], offset=tile_c * 256) as B_cols:
            with partition(C, p=block[1], offset=tile_r * 128 * N + tile_c * 256) as C_tile:
                with group(block[1]):
                    first: shared(float[12288], static=True) @ block[1]
                    second: shared(float[12288], static=True) @ block[1]
                    acc: float[64] @ thread[1] = {0}
                    for k0 in range(0, K, 64):
                        with claim(first, p=thread[256], offset=0) as first_fill:
                            with claim(second, p=thread[256], offset=0) as second_fill:
                                match split(thread):
                                    case 256:
                                        fill_slot_f32(first_fill, A_rows, B_cols, N, K, k0)
                                        fill_slot_f32(second_fill, A_rows, B_cols, N, K, k0 + 32)
                                    case 512:
                                        multiply_slot_f32(acc, first)
                                        multiply_slot_f32(acc, second)
                    with partition(C_tile, p=thread[1], offset=0) as C_mine:
                        match split(thread):
                            case 256:
                                pass
                            case 512:
                                wave: int @ thread[64] = id()
                                with group(thread[64]):
                                    lane: int @ thread[1] = id()
                                    with group(thread[1]):
                                        for i in range(2):
                                            for j in range(2):
                                                for v in range(16):
                                                    at: int @ thread[1] = (64 * (wave / 4) + 32 * i + 8 * (v / 4) + 4 * (lane / 32) + v % 4) * N \
                                                        + 64 * (wave % 4) + 32 * j + lane % 32
                                                    C_mine[at] = alpha * acc[(2 * i + j) * 16 + v] + beta * C_mine[at]
