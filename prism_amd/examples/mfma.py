"""One matrix instruction per wavefront and K step, operands straight from global memory: the teaching kernels
of examples/simple_mma.py and examples/mmaTF32NaiveKernel.py:14-85 on the matrix instructions of gfx950
(fp32 16x16x4, and bf16 16x16x32 with the operand layout of examples/h100_matmul.py: both operands K-contiguous).
"""
from prism_amd.hipgen import bf16, block, const, float4, float4_cast, grid, group, intrinsic, partition, prism, ptr, requires, thread


@requires(grid[1], block[1], thread[64])
@prism("global")
def one_mfma_per_wavefront(A: ptr(const(float)) @ grid[1], B: ptr(const(float)) @ grid[1], C: ptr(float) @ grid[1],
                           M: int @ grid[1], N: int @ grid[1], K: int @ grid[1]):
    """C = A B with one wavefront per 16 x 16 tile of C and one 16x16x4 fp32 MFMA per K step of 4, operands
    straight from global memory (the teaching kernel of examples/mmaTF32NaiveKernel.py:14-85, for whole tiles)."""
    tiles_n: const(int) @ grid[1] = N / 16
    w: const(int) @ thread[64] = id()
    tile_r: const(int) @ thread[64] = w / tiles_n
    tile_c: const(int) @ thread[64] = w % tiles_n
    with partition(A, p=thread[64], offset=tile_r * 16 * K) as A_rows:
        with partition(B, p=thread[64], offset=tile_c * 16) as B_cols:
            with partition(C, p=thread[64], offset=tile_r * 16 * N + tile_c * 16) as C_tile:
                with group(block[1]):
                    with group(thread[64]):
                        lane: const(int) @ thread[1] = id()
                        r: const(int) @ thread[1] = lane % 16
                        q: const(int) @ thread[1] = lane / 16
                        c0: float @ thread[1] = 0
                        c1: float @ thread[1] = 0
                        c2: float @ thread[1] = 0
                        c3: float @ thread[1] = 0
                        if w < (M / 16) * tiles_n:
                            for k0 in range(0, K, 4):
                                intrinsic.mfma_f32_16x16x4_f32(A_rows[r * K + k0 + q], B_cols[(k0 + q) * N + r],
                                                               c0, c1, c2, c3, out=[c0, c1, c2, c3])
                        with partition(C_tile, p=thread[1], offset=4 * q * N + r) as C_mine:
                            with group(thread[1]):
                                if w < (M / 16) * tiles_n:
                                    C_mine[0 * N] = c0
                                    C_mine[1 * N] = c1
                                    C_mine[2 * N] = c2
                                    C_mine[3 * N] = c3


@requires(grid[1], block[1], thread[64])
@prism("global")
def one_bf16_mfma_per_wavefront(P: ptr(const(bf16)) @ grid[1], Q: ptr(const(bf16)) @ grid[1], D: ptr(float) @ grid[1],
                                M: int @ grid[1], N: int @ grid[1], K: int @ grid[1]):
    """D = P Q^T (P is M x K, Q is N x K, both bf16 with K contiguous: the operand layout of
    examples/h100_matmul.py) with one wavefront per 16 x 16 tile of D and one 16x16x32 bf16 MFMA per K step of
    32; every lane fetches 16-byte packets of eight bf16 straight from global memory."""
    tiles_n: const(int) @ grid[1] = N / 16
    w: const(int) @ thread[64] = id()
    tile_r: const(int) @ thread[64] = w / tiles_n
    tile_c: const(int) @ thread[64] = w % tiles_n
    with partition(P, p=thread[64], offset=tile_r * 16 * K) as P_rows:
        with partition(Q, p=thread[64], offset=tile_c * 16 * K) as Q_rows:
            with partition(D, p=thread[64], offset=tile_r * 16 * N + tile_c * 16) as D_tile:
                with group(block[1]):
                    with group(thread[64]):
                        lane: const(int) @ thread[1] = id()
                        r: const(int) @ thread[1] = lane % 16
                        q: const(int) @ thread[1] = lane / 16
                        c0: float @ thread[1] = 0
                        c1: float @ thread[1] = 0
                        c2: float @ thread[1] = 0
                        c3: float @ thread[1] = 0
                        if w < (M / 16) * tiles_n:
                            for k0 in range(0, K, 32):
                                a: float4 @ thread[1] = float4_cast(P_rows[r * K + k0 + 8 * q])
                                b: float4 @ thread[1] = float4_cast(Q_rows[r * K + k0 + 8 * q])
                                intrinsic.mfma_f32_16x16x32_bf16(a, b, c0, c1, c2, c3, out=[c0, c1, c2, c3])
                        with partition(D_tile, p=thread[1], offset=4 * q * N + r) as D_mine:
                            with group(thread[1]):
                                if w < (M / 16) * tiles_n:
                                    D_mine[0 * N] = c0
                                    D_mine[1 * N] = c1
                                    D_mine[2 * N] = c2
                                    D_mine[3 * N] = c3
