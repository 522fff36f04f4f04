"""Every wavefront loads and multiplies: SGEMM on 256 x 256 tiles with two LDS stages and no written barrier.

The shape of the hand-written whole-tile kernel (prism_amd/csrc/sgemm.hip, sgemm_wave_tile_dma_kernel) in the
DSL: sixteen wavefronts own 32 x 128 strips of the tile in accumulators, a K tile of 32 travels from global
memory straight into LDS (`intrinsic.load_to_lds`, 64 lanes x 16 bytes per instruction), and while one stage is
multiplied the loads of the next K tile fill the other. The program only names who writes and who reads each
stage; the generator's access analysis puts one workgroup barrier in front of each refill and one at the end of
the loop body, i.e. one per K tile, and because a barrier waits for the wavefront's outstanding loads, a tile's
loads have a whole multiplication to land.

Stage layout (16384 floats): 256 rows of A with 32 k each (128-byte rows, the 16-byte chunk c of row r kept at
c ^ ((r / 2) % 8), which spreads a wavefront's operand reads over the banks), then 32 k-rows of B with 256
columns each (1 KiB rows, as in global memory).
"""
from prism_amd.hipgen import attr, bf16, block, const, float4, float4_cast, grid, group, intrinsic, partition, prism, ptr, requires, shared, thread


@requires(thread[1024])
@prism("device")
def fill_stage_f32(stage: ptr(float) @ block[1], A_from: ptr(const(float)) @ block[1], B_from: ptr(const(float)) @ block[1],
                   N: int @ grid[1], K: int @ grid[1], k_at: int @ block[1]):
    """Sixteen wavefronts start the copy of 256 rows x 32 k of A (eight rows per direct load) and of 32 k-rows x 256
    columns of B (one k-row per direct load): four loads per wavefront."""
    with group(thread[1024]):
        w: int @ thread[64] = id()
        with group(thread[64]):
            lane: int @ thread[1] = id()
            for part in range(2):
                arow: int @ thread[1] = 8 * (16 * part + w) + lane / 8
                intrinsic.load_to_lds(stage[256 * (16 * part + w)],
                                      A_from[arow * K + k_at + 4 * ((lane % 8) ^ ((arow / 2) % 8))])
            for part in range(2):
                intrinsic.load_to_lds(stage[8192 + 256 * (16 * part + w)], B_from[(k_at + 16 * part + w) * N + 4 * lane])
    return


@requires(thread[1024])
@prism("device")
def multiply_stage_f32(acc: ptr(float) @ thread[1], stage: ptr(const(float)) @ block[1]):
    """Sixteen wavefronts, eight down and two across, each adding its 32 x 128 strip of (A part)(B part) to acc.
    Operands come in 16-byte LDS reads: per group of 8 k a lane (l32, half) takes the chunk of 4 k values
    8 s + 4 half .. + 3 of its A row and, for each of those k, 4 consecutive B columns 4 l32 .. 4 l32 + 3.
    Instruction (jj, j) multiplies k = 8 s + jj (lower half-wavefront) and 8 s + 4 + jj (upper half) into
    sub-tile j, whose lane l32 thereby holds column 4 l32 + j:
    acc[j * 16 + v] = C[8 (v / 4) + 4 half + v % 4][4 l32 + j] of the strip."""
    with group(thread[1024]):
        wave: int @ thread[64] = id()
        row0: int @ thread[64] = 32 * (wave / 2)
        col0: int @ thread[64] = 128 * (wave % 2)
        with group(thread[64]):
            lane: int @ thread[1] = id()
            l32: int @ thread[1] = lane % 32
            half: int @ thread[1] = lane / 32
            a: float[4] @ thread[1]
            b: float[16] @ thread[1]
            for s in range(4):
                float4_cast[a[0]] = float4_cast(stage[(row0 + l32) * 32 + 4 * ((2 * s + half) ^ ((l32 / 2) % 8))])
                for jj in range(4):
                    float4_cast[b[4 * jj]] = float4_cast(stage[8192 + (8 * s + 4 * half + jj) * 256 + col0 + 4 * l32])
                for jj in range(4):
                    for j in range(4):
                        intrinsic.mfma_f32_32x32x2_f32(a[jj], b[4 * jj + j], acc[j * 16 + 0], acc[j * 16 + 1], acc[j * 16 + 2], acc[j * 16 + 3], acc[j * 16 + 4], acc[j * 16 + 5], acc[j * 16 + 6], acc[j * 16 + 7], acc[j * 16 + 8], acc[j * 16 + 9], acc[j * 16 + 10], acc[j * 16 + 11], acc[j * 16 + 12], acc[j * 16 + 13], acc[j * 16 + 14], acc[j * 16 + 15],
                                                       out=[acc[j * 16 + 0], acc[j * 16 + 1], acc[j * 16 + 2], acc[j * 16 + 3], acc[j * 16 + 4], acc[j * 16 + 5], acc[j * 16 + 6], acc[j * 16 + 7], acc[j * 16 + 8], acc[j * 16 + 9], acc[j * 16 + 10], acc[j * 16 + 11], acc[j * 16 + 12], acc[j * 16 + 13], acc[j * 16 + 14], acc[j * 16 + 15]])
    return


@attr("__launch_bounds__(1024)")
@requires(grid[1], block[1], thread[1024])
@prism("global")
def pipelined_sgemm(M: int @ grid[1], N: int @ grid[1], K: int @ grid[1], alpha: float @ grid[1],
                    A: ptr(const(float)) @ grid[1], B: ptr(const(float)) @ grid[1], beta: float @ grid[1],
                    C: ptr(float) @ grid[1], tiles_n: int @ grid[1]):
    """M a multiple of 2048, N of 256, K of 64; tiles_n = N / 256. Consecutive workgroups go to the eight XCDs in
    turn; each XCD walks its own band of tiles in columns of eight, so that its workgroups share panels in its L2."""
    per_xcd: const(int) @ block[1] = ((M / 256) * tiles_n) / 8
    t: const(int) @ block[1] = (id() % 8) * per_xcd + id() / 8
    tile_r: const(int) @ block[1] = 8 * (t / (8 * tiles_n)) + t % 8
    tile_c: const(int) @ block[1] = (t % (8 * tiles_n)) / 8
    with partition(A, p=block[1], offset=tile_r * 256 * K) as A_rows:
        with partition(B, p=block[1], offset=tile_c * 256) as B_cols:
            with partition(C, p=block[1], offset=tile_r * 256 * N + tile_c * 256) as C_tile:
                with group(block[1]):
                    first: shared(float[16384], static=True) @ block[1]
                    second: shared(float[16384], static=True) @ block[1]
                    acc: float[64] @ thread[1] = {0}
                    fill_stage_f32(first, A_rows, B_cols, N, K, 0)
                    for k0 in range(0, K, 64):
                        fill_stage_f32(second, A_rows, B_cols, N, K, k0 + 32)
                        multiply_stage_f32(acc, first)
                        if k0 + 64 < K:
                            fill_stage_f32(first, A_rows, B_cols, N, K, k0 + 64)
                        multiply_stage_f32(acc, second)
                    with partition(C_tile, p=thread[1], offset=0) as C_mine:
                        wave: int @ thread[64] = id()
                        with group(thread[64]):
                            lane: int @ thread[1] = id()
                            with group(thread[1]):
                                for v in range(16):
                                    for j in range(4):
                                        at: int @ thread[1] = (32 * (wave / 2) + 8 * (v / 4) + 4 * (lane / 32) + v % 4) * N \
                                            + 128 * (wave % 2) + 4 * (lane % 32) + j
                                        C_mine[at] = alpha * acc[j * 16 + v] + beta * C_mine[at]


# The bf16 product D = P Q^T (P is M x K, Q is N x K, K contiguous) the same way: eight wavefronts own 64 x 128
# parts of a 256 x 256 tile, a stage holds 64 k of both panels (256 rows of P, then 256 rows of Q, 128-byte rows
# with their 16-byte chunks swizzled as above), and the 16 x 16 x 32 matrix instruction takes 16-byte LDS reads.

@requires(thread[512])
@prism("device")
def fill_stage_bf16(stage: ptr(bf16) @ block[1], P_from: ptr(const(bf16)) @ block[1], Q_from: ptr(const(bf16)) @ block[1],
                    K: int @ grid[1], k_at: int @ block[1]):
    """Eight wavefronts start the copy of 256 rows x 64 k of P and of Q (eight rows per direct load): eight loads
    per wavefront."""
    with group(thread[512]):
        w: int @ thread[64] = id()
        with group(thread[64]):
            lane: int @ thread[1] = id()
            for part in range(4):
                prow: int @ thread[1] = 8 * (8 * part + w) + lane / 8
                intrinsic.load_to_lds(stage[512 * (8 * part + w)],
                                      P_from[prow * K + k_at + 8 * ((lane % 8) ^ ((prow / 2) % 8))])
            for part in range(4):
                qrow: int @ thread[1] = 8 * (8 * part + w) + lane / 8
                intrinsic.load_to_lds(stage[16384 + 512 * (8 * part + w)],
                                      Q_from[qrow * K + k_at + 8 * ((lane % 8) ^ ((qrow / 2) % 8))])
    return


@requires(thread[512])
@prism("device")
def multiply_stage_bf16(acc: ptr(float) @ thread[1], stage: ptr(const(bf16)) @ block[1]):
    """Eight wavefronts, four down and two across, each adding its 64 x 128 part of (P part)(Q part)^T to acc: two
    k-steps of 4 x 8 matrix instructions of 16 x 16 x 32;
    acc[(8 i + j) * 4 + v] = D[16 i + 4 (lane / 16) + v][16 j + lane % 16] of the part."""
    with group(thread[512]):
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
                    a[i] = float4_cast(stage[(row0 + 16 * i + r) * 64 + k8])
                for j in range(8):
                    b: float4 @ thread[1] = float4_cast(stage[16384 + (col0 + 16 * j + r) * 64 + k8])
                    for i in range(4):
                        intrinsic.mfma_f32_16x16x32_bf16(
                            a[i], b, acc[(8 * i + j) * 4], acc[(8 * i + j) * 4 + 1], acc[(8 * i + j) * 4 + 2], acc[(8 * i + j) * 4 + 3],
                            out=[acc[(8 * i + j) * 4], acc[(8 * i + j) * 4 + 1], acc[(8 * i + j) * 4 + 2], acc[(8 * i + j) * 4 + 3]])
    return


@attr("__launch_bounds__(512)")
@requires(grid[1], block[1], thread[512])
@prism("global")
def pipelined_gemm_bf16(P: ptr(const(bf16)) @ grid[1], Q: ptr(const(bf16)) @ grid[1], D: ptr(float) @ grid[1],
                        N: int @ grid[1], K: int @ grid[1], tiles_m: int @ grid[1], tiles_n: int @ grid[1]):
    """D = P Q^T on 256 x 256 tiles. K is a multiple of 128, M of 2048 and N of 256 (tiles_m = M / 256 a multiple of
    8, tiles_n = N / 256). Tile order as in pipelined_sgemm."""
    per_xcd: const(int) @ block[1] = (tiles_m * tiles_n) / 8
    t: const(int) @ block[1] = (id() % 8) * per_xcd + id() / 8
    tile_r: const(int) @ block[1] = 8 * (t / (8 * tiles_n)) + t % 8
    tile_c: const(int) @ block[1] = (t % (8 * tiles_n)) / 8
    with partition(P, p=block[1], offset=tile_r * 256 * K) as P_rows:
        with partition(Q, p=block[1], offset=tile_c * 256 * K) as Q_rows:
            with partition(D, p=block[1], offset=tile_r * 256 * N + tile_c * 256) as D_tile:
                with group(block[1]):
                    first: shared(bf16[32768], static=True) @ block[1]
                    second: shared(bf16[32768], static=True) @ block[1]
                    acc: float[128] @ thread[1] = {0}
                    fill_stage_bf16(first, P_rows, Q_rows, K, 0)
                    for k0 in range(0, K, 128):
                        # A fill and the multiplication behind it are one stretch of straight-line code, and the
                        # scheduling groups say how its instructions are to be interleaved: the 4 + 1 operand
                        # reads the first matrix instructions need, then groups of four matrix instructions with
                        # the next operand read and, in the first k-step, one of the fill's eight global loads
                        # behind each (a burst of loads holds the wavefront, and the matrix pipe with it, at the
                        # memory pipeline). Measured at 8192^3: 1156 TFLOP/s as the compiler orders it, 1280 so.
                        fill_stage_bf16(second, P_rows, Q_rows, K, k0 + 64)
                        multiply_stage_bf16(acc, first)
                        intrinsic.sched_group("lds_read", 5)
                        for g in range(7):
                            intrinsic.sched_group("mfma", 4)
                            intrinsic.sched_group("lds_read", 1)
                            intrinsic.sched_group("vmem_read", 1)
                        intrinsic.sched_group("mfma", 4)
                        intrinsic.sched_group("vmem_read", 1)
                        intrinsic.sched_group("lds_read", 5)
                        for g in range(7):
                            intrinsic.sched_group("mfma", 4)
                            intrinsic.sched_group("lds_read", 1)
                        intrinsic.sched_group("mfma", 4)
                        # The refill is not put under `if k0 + 128 < K`: a branch would end the stretch of code the
                        # groups order. The last trip fetches the first K tile once more, into a stage nobody
                        # reads again; the barrier at the end of the body waits for those loads as for all others.
                        fill_stage_bf16(first, P_rows, Q_rows, K, (k0 + 128) % K)
                        multiply_stage_bf16(acc, second)
                        intrinsic.sched_group("lds_read", 5)
                        for g in range(7):
                            intrinsic.sched_group("mfma", 4)
                            intrinsic.sched_group("lds_read", 1)
                            intrinsic.sched_group("vmem_read", 1)
                        intrinsic.sched_group("mfma", 4)
                        intrinsic.sched_group("vmem_read", 1)
                        intrinsic.sched_group("lds_read", 5)
                        for g in range(7):
                            intrinsic.sched_group("mfma", 4)
                            intrinsic.sched_group("lds_read", 1)
                        intrinsic.sched_group("mfma", 4)
                    with partition(D_tile, p=thread[1], offset=0) as D_mine:
                        wave: int @ thread[64] = id()
                        with group(thread[64]):
                            lane: int @ thread[1] = id()
                            with group(thread[1]):
                                for i in range(4):
                                    for j in range(8):
                                        for v in range(4):
                                            D_mine[(64 * (wave / 2) + 16 * i + 4 * (lane / 16) + v) * N
                                                   + 128 * (wave % 2) + 16 * j + lane % 16] = acc[(8 * i + j) * 4 + v]
