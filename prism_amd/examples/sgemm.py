"""SGEMM, C = alpha A B + beta C (row-major), in the steps of the reference's example set.

naive_sgemm        one thread per element of C (examples/sgemm_kernel_1.py)
remapped_sgemm     the same with a workgroup's threads laid over a 32 x 32 tile (examples/sgemm_kernel_2.py)
tiled_sgemm        TILE x TILE tiles of A and B staged in LDS (examples/sgemm_shared_mem_block.py)
thread_tile_sgemm  a TM x TN block of C per thread, operands in private arrays (examples/sgemm_kernel_3.py)
vector_tile_sgemm  16-byte global accesses, the A tile stored k-major (examples/sgemm_kernel_4.py)
staged_sgemm       the K step as two device functions that are handed the LDS tiles (examples/sgemm_kernel_5.py)
mfma_tile_sgemm    the same tiling with the product on the fp32 matrix instruction of gfx950, one 32 x 32 corner
                   per wavefront (no counterpart in the reference, whose fp32 kernels use no matrix instruction)

None of them places a barrier by hand. Tile sizes must divide the problem, as in the reference.
"""
from prism_amd.hipgen import attr, block, const, float4, float4_cast, grid, group, intrinsic, partition, prism, ptr, requires, shared, thread


@requires(grid[1], block[1], thread[1])
@prism("global")
def naive_sgemm(M: int @ grid[1], N: int @ grid[1], K: int @ grid[1], alpha: float @ grid[1],
                A: ptr(const(float)) @ grid[1], B: ptr(const(float)) @ grid[1], beta: float @ grid[1],
                C: ptr(float) @ grid[1], per_block: int @ grid[1]):
    blk: int @ block[1] = id()
    with partition(C, p=block[1], offset=0) as C_of_block:
        with group(block[1]):
            e: int @ thread[1] = blk * per_block + id()
            row: const(int) @ thread[1] = e / N
            col: const(int) @ thread[1] = e % N
            with partition(C_of_block, p=thread[1], offset=0) as C_mine:
                with group(thread[1]):
                    if e < M * N:
                        acc: float @ thread[1] = 0
                        for k in range(K):
                            acc += A[row * K + k] * B[k * N + col]
                        C_mine[row * N + col] = alpha * acc + beta * C_mine[row * N + col]


@requires(grid[1], block[1], thread[1])
@prism("global")
def remapped_sgemm(M: int @ grid[1], N: int @ grid[1], K: int @ grid[1], alpha: float @ grid[1],
                   A: ptr(const(float)) @ grid[1], B: ptr(const(float)) @ grid[1], beta: float @ grid[1],
                   C: ptr(float) @ grid[1], tiles_n: int @ grid[1]):
    """One thread per element with the 1024 threads of a workgroup laid over a 32 x 32 tile of C, consecutive
    threads along a row (examples/sgemm_kernel_2.py); guarded, so that M and N need not be multiples of 32."""
    tile_r: const(int) @ block[1] = id() / tiles_n
    tile_c: const(int) @ block[1] = id() % tiles_n
    with partition(C, p=block[1], offset=0) as C_of_block:
        with group(block[1]):
            t: int @ thread[1] = id()
            row: const(int) @ thread[1] = tile_r * 32 + t / 32
            col: const(int) @ thread[1] = tile_c * 32 + t % 32
            with partition(C_of_block, p=thread[1], offset=0) as C_mine:
                with group(thread[1]):
                    if row < M and col < N:
                        acc: float @ thread[1] = 0
                        for k in range(K):
                            acc += A[row * K + k] * B[k * N + col]
                        C_mine[row * N + col] = alpha * acc + beta * C_mine[row * N + col]


@requires(grid[1], block[1], thread[1])
@prism("global")
def tiled_sgemm(M: int @ grid[1], N: int @ grid[1], K: int @ grid[1], alpha: float @ grid[1],
                A: ptr(const(float)) @ grid[1], B: ptr(const(float)) @ grid[1], beta: float @ grid[1],
                C: ptr(float) @ grid[1], tiles_n: int @ grid[1], template=[("TILE", int)]):
    tile_r: const(int) @ block[1] = id() / tiles_n
    tile_c: const(int) @ block[1] = id() % tiles_n
    with partition(A, p=block[1], offset=tile_r * TILE * K) as A_rows:
        with partition(B, p=block[1], offset=tile_c * TILE) as B_cols:
            with partition(C, p=block[1], offset=tile_r * TILE * N + tile_c * TILE) as C_tile:
                with group(block[1]):
                    a_lds: shared(float[TILE * TILE], static=True) @ block[1]
                    b_lds: shared(float[TILE * TILE], static=True) @ block[1]
                    r: const(int) @ thread[1] = id() / TILE
                    c: const(int) @ thread[1] = id() % TILE
                    acc: float @ thread[1] = 0
                    for k0 in range(0, K, TILE):
                        with partition(a_lds, p=thread[1], offset=0) as a_mine:
                            with partition(b_lds, p=thread[1], offset=0) as b_mine:
                                with group(thread[1]):
                                    a_mine[r * TILE + c] = A_rows[r * K + k0 + c]
                                    b_mine[r * TILE + c] = B_cols[(k0 + r) * N + c]
                                    for d in range(TILE):
                                        acc += a_lds[r * TILE + d] * b_lds[d * TILE + c]
                    with partition(C_tile, p=thread[1], offset=r * N + c) as C_mine:
                        with group(thread[1]):
                            C_mine[0] = alpha * acc + beta * C_mine[0]


@attr("__launch_bounds__((BM * BN) / (TM * TN))")
@requires(grid[1], block[1], thread[1], smem=8192)
@prism("global")
def thread_tile_sgemm(M: int @ grid[1], N: int @ grid[1], K: int @ grid[1], alpha: float @ grid[1],
                      A: ptr(const(float)) @ grid[1], B: ptr(const(float)) @ grid[1], beta: float @ grid[1],
                      C: ptr(float) @ grid[1], tiles_n: int @ grid[1],
                      template=[("BM", int), ("BN", int), ("BK", int), ("TM", int), ("TN", int)]):
    tile_r: const(int) @ block[1] = id() / tiles_n
    tile_c: const(int) @ block[1] = id() % tiles_n
    with partition(A, p=block[1], offset=tile_r * BM * K) as A_rows:
        with partition(B, p=block[1], offset=tile_c * BN) as B_cols:
            with partition(C, p=block[1], offset=tile_r * BM * N + tile_c * BN) as C_tile:
                with group(block[1]):
                    a_lds: shared(float[1024]) @ block[1]
                    b_lds: shared(float[1024]) @ block[1]
                    t: const(int) @ thread[1] = id()
                    threads: const(int) @ thread[1] = (BM * BN) / (TM * TN)
                    out_r: const(int) @ thread[1] = t / (BN / TN)
                    out_c: const(int) @ thread[1] = t % (BN / TN)
                    acc: float[16] @ thread[1] = {0}
                    a_reg: float[4] @ thread[1] = {0}
                    b_reg: float[4] @ thread[1] = {0}
                    for k0 in range(0, K, BK):
                        with partition(a_lds, p=thread[1], offset=0) as a_mine:
                            with partition(b_lds, p=thread[1], offset=0) as b_mine:
                                with group(thread[1]):
                                    for e in range(t, BM * BK, threads):
                                        a_mine[e] = A_rows[(e / BK) * K + k0 + e % BK]
                                    for e in range(t, BK * BN, threads):
                                        b_mine[e] = B_cols[(k0 + e / BN) * N + e % BN]
                                    for kk in range(BK):
                                        for i in range(TM):
                                            a_reg[i] = a_lds[(out_r * TM + i) * BK + kk]
                                        for j in range(TN):
                                            b_reg[j] = b_lds[kk * BN + out_c * TN + j]
                                        for i in range(TM):
                                            for j in range(TN):
                                                acc[i * TN + j] += a_reg[i] * b_reg[j]
                    with partition(C_tile, p=thread[1], offset=out_r * TM * N + out_c * TN) as C_mine:
                        with group(thread[1]):
                            for i in range(TM):
                                for j in range(TN):
                                    C_mine[i * N + j] = alpha * acc[i * TN + j] + beta * C_mine[i * N + j]


@attr("__launch_bounds__((BM * BN) / (TM * TN))")
@requires(grid[1], block[1], thread[1], smem=8192)
@prism("global")
def vector_tile_sgemm(M: int @ grid[1], N: int @ grid[1], K: int @ grid[1], alpha: float @ grid[1],
                      A: ptr(float) @ grid[1], B: ptr(float) @ grid[1], beta: float @ grid[1],
                      C: ptr(float) @ grid[1], tiles_n: int @ grid[1],
                      template=[("BM", int), ("BN", int), ("BK", int), ("TM", int), ("TN", int)]):
    """Thread-tile SGEMM with 16-byte global loads and stores; the A tile is stored transposed (BK x BM)
    through an index-mapped view, so that a K slice of it is contiguous. One packet of A and one of B per
    thread: BM * BK = BK * BN = 4 * threads."""
    tile_r: const(int) @ block[1] = id() / tiles_n
    tile_c: const(int) @ block[1] = id() % tiles_n
    with partition(A, p=block[1], offset=tile_r * BM * K) as A_rows:
        with partition(B, p=block[1], offset=tile_c * BN) as B_cols:
            with partition(C, p=block[1], offset=tile_r * BM * N + tile_c * BN) as C_tile:
                with group(block[1]):
                    a_lds: shared(float[1024]) @ block[1]
                    b_lds: shared(float[1024]) @ block[1]
                    t: const(int) @ thread[1] = id()
                    out_r: const(int) @ thread[1] = t / (BN / TN)
                    out_c: const(int) @ thread[1] = t % (BN / TN)
                    a_row: const(int) @ thread[1] = t / (BK / 4)
                    a_quad: const(int) @ thread[1] = t % (BK / 4)
                    b_row: const(int) @ thread[1] = t / (BN / 4)
                    b_quad: const(int) @ thread[1] = t % (BN / 4)
                    acc: float[64] @ thread[1] = {0}
                    a_reg: float[8] @ thread[1] = {0}
                    b_reg: float[8] @ thread[1] = {0}
                    for k0 in range(0, K, BK):
                        with partition(a_lds, p=thread[1], f=lambda e: (e % BK) * BM + e / BK) as a_by_row:
                            with group(thread[1]):
                                quad: float4 @ thread[1] = float4_cast(A_rows[a_row * K + k0 + a_quad * 4])
                                a_by_row[a_row * BK + a_quad * 4] = quad.x
                                a_by_row[a_row * BK + a_quad * 4 + 1] = quad.y
                                a_by_row[a_row * BK + a_quad * 4 + 2] = quad.z
                                a_by_row[a_row * BK + a_quad * 4 + 3] = quad.w
                                float4_cast[b_lds[b_row * BN + b_quad * 4]] = \
                                    float4_cast(B_cols[(k0 + b_row) * N + b_quad * 4])
                                for kk in range(BK):
                                    for i in range(TM):
                                        a_reg[i] = a_lds[kk * BM + out_r * TM + i]
                                    for j in range(TN):
                                        b_reg[j] = b_lds[kk * BN + out_c * TN + j]
                                    for i in range(TM):
                                        for j in range(TN):
                                            acc[i * TN + j] += a_reg[i] * b_reg[j]
                    for i in range(TM):
                        for j in range(0, TN, 4):
                            with partition(C_tile, p=thread[1], offset=(out_r * TM + i) * N + out_c * TN + j) as c4:
                                with group(thread[1]):
                                    was: float4 @ thread[1] = float4_cast(c4[0])
                                    was.x = alpha * acc[i * TN + j] + beta * was.x
                                    was.y = alpha * acc[i * TN + j + 1] + beta * was.y
                                    was.z = alpha * acc[i * TN + j + 2] + beta * was.z
                                    was.w = alpha * acc[i * TN + j + 3] + beta * was.w
                                    float4_cast[c4[0]] = was


@requires(block[1], thread[1])
@prism("device")
def stage_tiles(N: int @ grid[1], K: int @ grid[1], A_from: ptr(const(float)) @ block[1], B_from: ptr(const(float)) @ block[1],
                a_tile: ptr(float) @ block[1], b_tile: ptr(float) @ block[1],
                template=[("BM", int), ("BN", int), ("BK", int), ("THREADS", int)]):
    """Copies a BM x BK tile of A (stored k-major) and a BK x BN tile of B into LDS, THREADS elements at a time."""
    with group(block[1]):
        t: const(int) @ thread[1] = id()
        with partition(a_tile, p=thread[1], offset=0) as a_mine:
            with partition(b_tile, p=thread[1], offset=0) as b_mine:
                with group(thread[1]):
                    for e in range(t, BM * BK, THREADS):
                        a_mine[(e % BK) * BM + e / BK] = A_from[(e / BK) * K + e % BK]
                    for e in range(t, BK * BN, THREADS):
                        b_mine[e] = B_from[(e / BN) * N + e % BN]
    return


@requires(block[1], thread[1])
@prism("device")
def multiply_tiles(acc: ptr(float) @ thread[1], a_tile: ptr(const(float)) @ block[1], b_tile: ptr(const(float)) @ block[1],
                   out_r: int @ thread[1], out_c: int @ thread[1],
                   template=[("BM", int), ("BN", int), ("BK", int), ("TM", int), ("TN", int)]):
    """acc (TM x TN, private) += the thread's rows of the A tile times its columns of the B tile."""
    with group(block[1]):
        with group(thread[1]):
            for kk in range(BK):
                for i in range(TM):
                    for j in range(TN):
                        acc[i * TN + j] += a_tile[kk * BM + out_r * TM + i] * b_tile[kk * BN + out_c * TN + j]
    return


@attr("__launch_bounds__(THREADS)")
@requires(grid[1], block[1], thread[1], smem=8192)
@prism("global")
def staged_sgemm(M: int @ grid[1], N: int @ grid[1], K: int @ grid[1], alpha: float @ grid[1],
                 A: ptr(const(float)) @ grid[1], B: ptr(const(float)) @ grid[1], beta: float @ grid[1],
                 C: ptr(float) @ grid[1], tiles_n: int @ grid[1],
                 template=[("BM", int), ("BN", int), ("BK", int), ("TM", int), ("TN", int), ("THREADS", int)]):
    """The K step as two device functions that are handed the LDS tiles, one filling and one reading them
    (the decomposition of examples/sgemm_kernel_5.py:12-57,103-113): the barriers between and behind them come
    from what the callees' signatures say about their pointer parameters."""
    tile_r: const(int) @ block[1] = id() / tiles_n
    tile_c: const(int) @ block[1] = id() % tiles_n
    with partition(A, p=block[1], offset=tile_r * BM * K) as A_rows:
        with partition(B, p=block[1], offset=tile_c * BN) as B_cols:
            with partition(C, p=block[1], offset=tile_r * BM * N + tile_c * BN) as C_tile:
                with group(block[1]):
                    a_lds: shared(float[1024]) @ block[1]
                    b_lds: shared(float[1024]) @ block[1]
                    t: const(int) @ thread[1] = id()
                    out_r: const(int) @ thread[1] = t / (BN / TN)
                    out_c: const(int) @ thread[1] = t % (BN / TN)
                    acc: float[16] @ thread[1] = {0}
                    for k0 in range(0, K, BK):
                        with partition(A_rows, p=block[1], offset=k0) as A_now:
                            with partition(B_cols, p=block[1], offset=k0 * N) as B_now:
                                stage_tiles(N, K, A_now, B_now, a_lds, b_lds, template=[BM, BN, BK, THREADS])
                                multiply_tiles(acc, a_lds, b_lds, out_r, out_c, template=[BM, BN, BK, TM, TN])
                    with partition(C_tile, p=thread[1], offset=out_r * TM * N + out_c * TN) as C_mine:
                        with group(thread[1]):
                            for i in range(TM):
                                for j in range(TN):
                                    C_mine[i * N + j] = alpha * acc[i * TN + j] + beta * C_mine[i * N + j]


@attr("__launch_bounds__(256)")
@requires(grid[1], block[1], thread[64])
@prism("global")
def mfma_tile_sgemm(M: int @ grid[1], N: int @ grid[1], K: int @ grid[1], alpha: float @ grid[1],
                    A: ptr(const(float)) @ grid[1], B: ptr(const(float)) @ grid[1], beta: float @ grid[1],
                    C: ptr(float) @ grid[1], tiles_n: int @ grid[1]):
    """C = alpha A B + beta C with 64 x 64 x 8 tiles staged in LDS and the product on fp32 MFMA: four wavefronts
    per workgroup, each owning a 32 x 32 corner in sixteen accumulators, one 32x32x2 instruction per pair of k
    values (the wave-level tiling of examples/sgemm_kernel_5.py with the matrix instruction in place of its
    per-thread loops). A is stored k-major so that both operands are read along a row of LDS."""
    tile_r: const(int) @ block[1] = id() / tiles_n
    tile_c: const(int) @ block[1] = id() % tiles_n
    with partition(A, p=block[1], offset=tile_r * 64 * K) as A_rows:
        with partition(B, p=block[1], offset=tile_c * 64) as B_cols:
            with partition(C, p=block[1], offset=tile_r * 64 * N + tile_c * 64) as C_tile:
                with group(block[1]):
                    a_lds: shared(float[512], static=True) @ block[1]
                    b_lds: shared(float[512], static=True) @ block[1]
                    t: const(int) @ thread[1] = id()
                    wave: const(int) @ thread[64] = id()
                    corner_r: const(int) @ thread[64] = (wave / 2) * 32
                    corner_c: const(int) @ thread[64] = (wave % 2) * 32
                    with partition(a_lds, p=thread[1], offset=0) as a_mine:
                        with partition(b_lds, p=thread[1], offset=0) as b_mine:
                            with partition(C_tile, p=thread[1], offset=0) as C_mine:
                                with group(thread[64]):
                                    lane: const(int) @ thread[1] = id()
                                    r: const(int) @ thread[1] = lane % 32
                                    q: const(int) @ thread[1] = lane / 32
                                    acc: float[16] @ thread[1] = {0}
                                    with group(thread[1]):
                                        for k0 in range(0, K, 8):
                                            for e in range(t, 512, 256):
                                                a_mine[(e % 8) * 64 + e / 8] = A_rows[(e / 8) * K + k0 + e % 8]
                                                b_mine[e] = B_cols[(k0 + e / 64) * N + e % 64]
                                            for kk in range(0, 8, 2):
                                                intrinsic.mfma_f32_32x32x2_f32(
                                                    a_lds[(kk + q) * 64 + corner_r + r], b_lds[(kk + q) * 64 + corner_c + r],
                                                    acc[0], acc[1], acc[2], acc[3], acc[4], acc[5], acc[6], acc[7],
                                                    acc[8], acc[9], acc[10], acc[11], acc[12], acc[13], acc[14], acc[15],
                                                    out=[acc[0], acc[1], acc[2], acc[3], acc[4], acc[5], acc[6], acc[7],
                                                         acc[8], acc[9], acc[10], acc[11], acc[12], acc[13], acc[14], acc[15]])
                                        for v in range(16):
                                            C_mine[(corner_r + 8 * (v / 4) + 4 * q + v % 4) * N + corner_c + r] = \
                                                alpha * acc[v] + beta * C_mine[(corner_r + 8 * (v / 4) + 4 * q + v % 4) * N + corner_c + r]
