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
from prism_amd.hipgen import bf16, block, claim, const, float4, float4_cast, grid, group, intrinsic, partition, prism, ptr, requires, shared, split, thread


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
