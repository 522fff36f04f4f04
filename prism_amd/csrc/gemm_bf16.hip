// bf16 x bf16 -> fp32-accumulate GEMM on MFMA: OUT[r][c] = sum_k P[r][k] * Q[c][k],
// P is R x K and Q is Cn x K, both row-major bf16 (K contiguous), OUT row-major.
//
// This is the gfx950 counterpart of the reference's Hopper kernel
// (examples/h100_matmul.py:20-297, generated/cutlass_my_h100_match_no_tail.cu):
//   reference                                   here
//   wgmma m64n256k16 from swizzled smem     ->  v_mfma_f32_16x16x32_bf16 (32x32x16 in the small-tile and
//                                               general kernels), 4 waves x 128x128, swizzled LDS
//   TMA bulk copies + mbarrier ring (4 x)   ->  direct-to-LDS loads two K tiles ahead into two LDS stages,
//                                               a stage freed in mid-phase once its fragments are in
//                                               registers (gemm_bf16_early_kernel); odd or small K tile
//                                               counts: direct-to-LDS ring of two stages
//                                               (gemm_bf16_ring_kernel)
//   1 producer + 2 consumer warpgroups      ->  every wave loads and multiplies
//   persistent CTAs + 16x8 super-tiles      ->  with more tiles than CUs one workgroup per CU that walks
//                                               its tiles and fetches the next tile's first K tiles in
//                                               the last phases of the current one, else one workgroup
//                                               per tile; 16x16 super-blocks with an 8x4 patch per XCD
//                                               (tile_map.h)
//   epilogue: registers -> global           ->  whole tiles leave as 256 B runs of rows through a wave's
//                                               own LDS patch, bf16 converted in hardware; a few rows or
//                                               columns beyond whole tiles run as strips
//                                               (gemm_bf16_thin_kernel)
//   K tail dropped, M/N multiples required  ->  any M, N, K. Ragged M, N, K with K a multiple of 8
//                                               (16 B-aligned rows): the same kernels, edges zero-filled
//                                               by the buffer loads' range check. K not a multiple of 8
//                                               or operands not 16 B aligned: the same kernels' ragged
//                                               forms (16 B loads from 2 B-aligned addresses, the last
//                                               K % 8 values of k added on the way out). K < 8 and
//                                               offsets beyond 32 bits: gemm_bf16_kernel (guarded
//                                               loads, 16 B where a packet lies inside its row; staged
//                                               in registers one K step ahead, padded LDS rows)
//
// prism_gemm_bf16 calls it with (P, Q) = (A, B) and an fp32 OUT = D[M][N].
// prism_runmyh100 needs the reference's column-major bf16 C (C[n * M + m],
// generated/cutlass_my_h100_match_no_tail.cu:313,347-354); that is the row-major
// N x M matrix B @ A^T, so it calls the same kernel with (P, Q) = (B, A) and a
// bf16 OUT, which keeps the stores contiguous.
//
// MFMA operand layout (both operands are "row x 8 consecutive k"): lane l holds
// P[r = l % 32][k = 8 * (l / 32) .. + 7] and Q[c = l % 32][same k]; result
// register v of lane l is OUT[8 * (v / 4) + 4 * (l / 32) + v % 4][l % 32].
//
// In gemm_bf16_kernel LDS rows are BK + 8 elements (144 B for BK = 64): eight lanes
// reading 16 B from eight consecutive rows then cover all banks exactly once.
#include <type_traits>

#include "common.h"
#include "direct_load.h"
#include "tile_map.h"

// gemm_bf16_early_kernel: K tiles (of 128 B) between the starting points of two XCDs' walks along K.
// 8192 x 8192 x K, TFLOP/s all starting at 0 / with 64: K = 12288 1316 / 1427, 6144 1432 / 1495, 10240 1436 / 1502,
// 14336 1507 / 1522, 8192 and 4096 level, 24576 1302 / 1273. Steps of 2 and 8 tiles (256 B, 1 KB) gain nothing,
// 16 half of it, 32 the same; at K = 12288 steps of 48, 96, 128 tiles and of half the K tiles give 1395, 1366,
// 1420, 1345 against 1435 for 64.
constexpr int kEarlyKStagger = 64;
// gemm_bf16_early_kernel: matrix instructions of a phase before the barrier that frees its stage, and between two
// direct loads. Barrier position / gap, PFLOP/s at 8192^3 and 16384^3: 64/2 1.33-1.37, 1.32; 64/4 1.41-1.42, 1.42;
// 48/5 1.43-1.44, 1.47; 40/5 1.44-1.45, 1.47; 36/6 1.44, 1.49. A wave-wide 16 B load keeps the CU's vector memory
// path busy for 16 clocks, and the 64 loads of a K tile are half of a phase's clocks: the more evenly they are
// spread, the less they hold up the matrix instructions behind them.
constexpr int kEarlyBarrierAt = 36, kEarlyLoadGap = 6;

namespace prism {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// fp32 -> bf16, round to nearest even; NaN stays NaN. gfx950 converts in hardware, two values per instruction
// (v_cvt_pk_bf16_f32); in integer arithmetic it is seven instructions per value, which for a 128 x 128 wave tile was
// 4 us of vector ALU work per tile with the matrix pipe idle.
__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) {
    return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
}

__device__ __forceinline__ void store_out(float* p, float v) { *p = v; }
__device__ __forceinline__ void store_out(uint16_t* p, float v) { *p = f32_to_bf16_rne(v); }

// Scheduling recipe for one k-substep of MFMAS matrix instructions:
// READS x {LDS read, MFMA}, then max(WRITES, LOADS) x {LDS write, global load, MFMA},
// then the remaining MFMAs back to back.
template <int N, typename F>
__device__ __forceinline__ void repeat(F&& f) {
    if constexpr (N > 0) {
        f();
        repeat<N - 1>(f);
    }
}
template <int READS, int WRITES, int LOADS, int MFMAS>
__device__ __forceinline__ void sched_substep() {
    constexpr int SLOTS = WRITES > LOADS ? WRITES : LOADS;
    constexpr int PAIRED = READS < MFMAS ? READS : MFMAS;
    constexpr int SLOT_MFMAS = (MFMAS - PAIRED) < SLOTS ? (MFMAS - PAIRED) : SLOTS;
    constexpr int REST = MFMAS - PAIRED - SLOT_MFMAS;
    repeat<PAIRED>([] {
        __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // LDS read
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
    });
    if constexpr (READS > PAIRED) __builtin_amdgcn_sched_group_barrier(0x100, READS - PAIRED, 0);
    repeat<SLOT_MFMAS>([] {
        if constexpr (WRITES > 0) __builtin_amdgcn_sched_group_barrier(0x200, (WRITES + SLOT_MFMAS - 1) / (SLOT_MFMAS > 0 ? SLOT_MFMAS : 1), 0);
        if constexpr (LOADS > 0) __builtin_amdgcn_sched_group_barrier(0x020, (LOADS + SLOT_MFMAS - 1) / (SLOT_MFMAS > 0 ? SLOT_MFMAS : 1), 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    });
    if constexpr (REST > 0) __builtin_amdgcn_sched_group_barrier(0x008, REST, 0);
}

template <int BM, int BN, int BK, int WM, int WN, bool EDGE, typename OutT>
__global__ __launch_bounds__((BM / WM) * (BN / WN) * kWave) void gemm_bf16_kernel(
    int R, int Cn, int K, const uint16_t* __restrict__ P, const uint16_t* __restrict__ Q,
    OutT* __restrict__ OUT, int tiles_m, int tiles_n) {
    constexpr int WAVES_N = BN / WN;
    constexpr int THREADS = (BM / WM) * WAVES_N * kWave;
    constexpr int MI = WM / 32, NI = WN / 32;
    constexpr int LD = BK + 8;                // LDS row length in elements
    constexpr int KP = BK / 8;                // 16 B packets per row
    constexpr int P_PACKETS = BM * KP, Q_PACKETS = BN * KP;
    static_assert(P_PACKETS % THREADS == 0 && Q_PACKETS % THREADS == 0, "whole packets per thread");
    constexpr int P_PER = P_PACKETS / THREADS, Q_PER = Q_PACKETS / THREADS;
    static_assert(BK % 16 == 0 && WM % 32 == 0 && WN % 32 == 0, "tile shapes");
    constexpr int P_TILE = BM * LD, Q_TILE = BN * LD;  // elements per buffer

    extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
    uint16_t* Ps = reinterpret_cast<uint16_t*>(smem_raw);  // [2][BM][LD]
    uint16_t* Qs = Ps + 2 * P_TILE;                        // [2][BN][LD]

    int tm, tn;
    xcd_tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn);
    const int row0 = tm * BM, col0 = tn * BN;

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1), wave = tid / kWave;
    const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;
    const int l32 = lane & 31, lhi = lane >> 5;

    f32x16 acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    u32x4 p_stage[P_PER], q_stage[Q_PER];

    // One 16 B packet = 8 consecutive k of one row.
    auto load_packet = [&](const uint16_t* base, int rows, int row, int k) -> u32x4 {
        if constexpr (!EDGE) {
            return *reinterpret_cast<const u32x4*>(&base[static_cast<size_t>(row) * K + k]);
        } else {
            u32x4 r = {0u, 0u, 0u, 0u};
            if (row < rows && k + 8 <= K) {
                // Whole packet inside the row: one 16 B access (rows may be only 2 B aligned).
                __builtin_memcpy(&r, &base[static_cast<size_t>(row) * K + k], 16);
            } else if (row < rows && k < K) {
                // The packet that straddles the end of the row: element by element.
                uint16_t e[8];
#pragma unroll
                for (int c = 0; c < 8; ++c) e[c] = (k + c < K) ? base[static_cast<size_t>(row) * K + k + c] : uint16_t{0};
#pragma unroll
                for (int c = 0; c < 4; ++c) r[c] = static_cast<uint32_t>(e[2 * c]) | (static_cast<uint32_t>(e[2 * c + 1]) << 16);
            }
            return r;
        }
    };
    auto load_global = [&](int k0) {
#pragma unroll
        for (int u = 0; u < P_PER; ++u) {
            const int p = tid + u * THREADS;
            p_stage[u] = load_packet(P, R, row0 + p / KP, k0 + (p % KP) * 8);
        }
#pragma unroll
        for (int u = 0; u < Q_PER; ++u) {
            const int p = tid + u * THREADS;
            q_stage[u] = load_packet(Q, Cn, col0 + p / KP, k0 + (p % KP) * 8);
        }
    };
    auto store_lds = [&](int buf) {
#pragma unroll
        for (int u = 0; u < P_PER; ++u) {
            const int p = tid + u * THREADS;
            *reinterpret_cast<u32x4*>(&Ps[buf * P_TILE + (p / KP) * LD + (p % KP) * 8]) = p_stage[u];
        }
#pragma unroll
        for (int u = 0; u < Q_PER; ++u) {
            const int p = tid + u * THREADS;
            *reinterpret_cast<u32x4*>(&Qs[buf * Q_TILE + (p / KP) * LD + (p % KP) * 8]) = q_stage[u];
        }
    };

    // Software pipeline, three K tiles in flight:
    //   LDS[buf]      tile t     being multiplied,
    //   LDS[buf ^ 1]  tile t+1   written from the staging registers at the top of step t,
    //   registers     tile t+2   global loads issued right after those writes.
    // MFMA operands are double-buffered too: the LDS reads of k-substep kk+1 are
    // issued before the MFMAs of substep kk.
    constexpr int KS = BK / 16;  // k-substeps (one MFMA depth each) per tile
    static_assert(KS % 2 == 0, "operand double-buffering assumes an even number of k-substeps");
    bf16x8 fa[2][MI], fb[2][NI];
    auto read_frags = [&](int buf, int kk, int slot) {
        const uint16_t* ps = &Ps[buf * P_TILE + (wave_m * WM + l32) * LD + lhi * 8 + kk * 16];
        const uint16_t* qs = &Qs[buf * Q_TILE + (wave_n * WN + l32) * LD + lhi * 8 + kk * 16];
#pragma unroll
        for (int i = 0; i < MI; ++i)
            fa[slot][i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(&ps[i * 32 * LD]));
#pragma unroll
        for (int j = 0; j < NI; ++j)
            fb[slot][j] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(&qs[j * 32 * LD]));
    };

    // One K tile. STORE: tile t+1 is waiting in the staging registers and goes
    // to the other LDS buffer; LOAD: tile t+2 exists and is fetched. The two
    // flags are compile-time so that the steady-state body is one basic block
    // the scheduler can interleave.
    auto k_step = [&](int t, auto store_next, auto load_next2) {
        const int buf = t & 1;
        if constexpr (store_next) store_lds(buf ^ 1);
        if constexpr (load_next2) load_global((t + 2) * BK);
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) {
            if (kk + 1 < KS) read_frags(buf, kk + 1, (kk + 1) & 1);
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < NI; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[kk & 1][i], fb[kk & 1][j], acc[i][j], 0, 0, 0);
        }
        // Issue order for the whole step: LDS reads of the next k-substep ride
        // under the first MFMAs of each substep, LDS writes and global loads of
        // the following tiles under the rest, so the matrix pipe never waits for
        // a burst of memory instructions to issue.
        constexpr int WRITES = store_next ? (P_PER + Q_PER) : 0;  // per step
        constexpr int LOADS = load_next2 ? (P_PER + Q_PER) : 0;
        constexpr int W_PER = (WRITES + KS - 1) / KS, L_PER = (LOADS + KS - 1) / KS;
#pragma unroll
        for (int kk = 0; kk < KS; ++kk) {
            if (kk + 1 < KS)
                sched_substep<MI + NI, W_PER, L_PER, MI * NI>();
            else
                sched_substep<0, W_PER, L_PER, MI * NI>();
        }
        __syncthreads();
        if constexpr (store_next) read_frags(buf ^ 1, 0, 0);
    };
    using yes = std::integral_constant<bool, true>;
    using no = std::integral_constant<bool, false>;

    const int k_tiles = (K + BK - 1) / BK;
    load_global(0);
    store_lds(0);
    if (k_tiles > 1) load_global(BK);
    __syncthreads();
    if (k_tiles > 0) read_frags(0, 0, 0);

    int t = 0;
    for (; t + 2 < k_tiles; ++t) k_step(t, yes{}, yes{});
    if (t + 1 < k_tiles) { k_step(t, yes{}, no{}); ++t; }
    if (t < k_tiles) k_step(t, no{}, no{});

#pragma unroll
    for (int i = 0; i < MI; ++i) {
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            const int col = col0 + wave_n * WN + j * 32 + l32;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = row0 + wave_m * WM + i * 32 + 8 * (v / 4) + 4 * lhi + (v % 4);
                if (!EDGE || (row < R && col < Cn))
                    store_out(&OUT[static_cast<size_t>(row) * Cn + col], acc[i][j][v]);
            }
        }
    }
}

// The last K_all - K (< 8) values of k of one row, for the kernels' ragged forms, whose K loops stop at K, a
// multiple of 8: the row's tail is one 16 B chunk (k = K .. K + 7, its end the head of the next row), fetched
// with a range-checked buffer load so that nothing past the matrix is touched; slots beyond the tail and rows
// beyond the matrix become zeros. The range check works on dwords: with an odd tail the very last element of
// the matrix shares its dword with what lies beyond and arrives as zero, so it is fetched again on its own.
// `first`: the tile's first row (the descriptor starts there: offsets stay small), `rows`: the matrix's row count.
__device__ __forceinline__ void load_k_tail(const uint16_t* base, int ld, int first, int rows, int row, int K, int K_all,
                                            float (&out)[7]) {
    auto as_float = [](uint32_t bits16) { return __builtin_bit_cast(float, bits16 << 16); };
    const int tail = K_all - K;
    const long long left = static_cast<long long>(rows - first) * ld * 2;
    const auto rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<uint16_t*>(base + (left > 0 ? static_cast<size_t>(first) * ld : size_t{0})), 0,
        static_cast<int>(clamped_extent(left)), 0x00020000);
    const u32x4 c = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(
        rsrc, (static_cast<uint32_t>(row - first) * static_cast<uint32_t>(ld) + static_cast<uint32_t>(K)) * 2u, 0, 0));
    const bool last_of_matrix = (tail & 1) && row == rows - 1;
    const float last = last_of_matrix ? as_float(base[static_cast<size_t>(row) * ld + K_all - 1]) : 0.0f;
#pragma unroll
    for (int t = 0; t < 7; ++t) {
        const uint32_t bits = (t & 1) ? (c[t / 2] >> 16) : (c[t / 2] & 0xffffu);
        out[t] = (t < tail && row < rows) ? as_float(bits) : 0.0f;
        if (last_of_matrix && t == tail - 1) out[t] = last;
    }
}

// ------------------------------------------------- direct-to-LDS ring kernel --
// Whole tiles, K a multiple of BK and at least STAGES K tiles. Global data goes
// straight into LDS (global_load_lds_dwordx4: no staging registers, no LDS write
// instructions), the role TMA plays in the reference
// (evals/h100_bench/utils.cuh:238-273). K tiles travel through a ring of STAGES
// LDS stages; the direct loads of tile t + STAGES - 1 are issued while tile t is
// multiplied, into the stage tile t-1 has just left.
//
// A wave-wide direct load writes 1 KiB of contiguous LDS (lane l lands at
// base + 16 l), so rows cannot be padded. Bank conflicts are avoided the way the
// reference's 128 B swizzle does it (utils.cuh:6-16): the 16 B chunk c of row r
// sits in slot c ^ ((r >> SWZ) & (chunks_per_row - 1)); the load side applies the
// permutation to the global address, the operand reads to the LDS address.
//
// With one wave per SIMD nothing hides a stall and every vector ALU instruction a
// wave issues between two MFMAs delays the second one, so the K loop is laid out
// by hand and pinned with scheduling barriers: MFMA, one LDS read, MFMA, one LDS
// read, ...; the operands of a group of 16 MFMAs are read behind the first half
// of the group before it; loads use a scalar base and a fixed lane offset (no
// vector ALU work in the loop).
//
// 64 x 2 stages is the shape used, for the K tile counts gemm_bf16_early_kernel below
// does not take: a direct load cannot be issued before its stage is free, so it has
// less than one tile time to land, which the early-read kernel avoids. 32 x 4 stages
// (also supported by the template) gives loads three tile times but reads half cache
// lines (64 B per row and tile) and measured slower than both.
//
// EDGE: M, N, K need not be whole tiles (K a multiple of 8, so that rows stay 16 B aligned and a
// 16 B chunk is whole or absent). The direct loads then go through buffer descriptors whose extents
// end with the matrices: rows beyond them arrive as zeros. Columns k >= K of a row are the next
// row's data, so in the partial K tile those lanes use an offset beyond any extent; the K loop
// runs over at least STAGES tiles, those beyond K all zeros.
//
// RAGGED (with EDGE): K need not be a multiple of 8 and P, Q need only be 2 B aligned (16 B loads from 2 B-
// aligned addresses); the K loop covers K rounded down to a multiple of 8 and the rest is added on the way out.
template <int BM, int BN, int BK, int STAGES, int WM, int WN, bool EDGE, typename OutT, bool RAGGED = false>
__global__ __launch_bounds__((BM / WM) * (BN / WN) * kWave) void gemm_bf16_ring_kernel(
    int R, int Cn, int K_all, const uint16_t* __restrict__ P, const uint16_t* __restrict__ Q,
    OutT* __restrict__ OUT, int tiles_m, int tiles_n, int first_big) {
    static_assert(EDGE || !RAGGED, "the ragged form is an edge form");
    const int ld = K_all;                                        // elements between rows of P and of Q
    const int K = RAGGED ? K_all - K_all % 8 : K_all;            // the part of the k range the loop covers
    static_assert((BK == 32 || BK == 64) && (STAGES == 2 || STAGES == 4), "ring shape");
    constexpr int KP = BK / 8;                        // 16 B chunks per row
    constexpr int SWZ = KP == 4 ? 2 : 1;
    constexpr int KS = BK / 16;                       // k-groups (one MFMA deep) per tile
    constexpr int AHEAD = STAGES - 1;                 // tiles in flight ahead of the one being multiplied
    constexpr int WAVES_N = BN / WN;
    constexpr int WAVES = (BM / WM) * WAVES_N;
    constexpr int MI = WM / 32, NI = WN / 32;
    constexpr int ROWS_PER_LOAD = kWave / KP;         // rows one wave-wide load covers
    constexpr int ROWS_PER_PASS = ROWS_PER_LOAD * WAVES;
    static_assert(BM % ROWS_PER_PASS == 0 && BN % ROWS_PER_PASS == 0, "whole load passes");
    constexpr int P_PER = BM / ROWS_PER_PASS, Q_PER = BN / ROWS_PER_PASS;  // loads per wave per tile
    constexpr int LOADS = P_PER + Q_PER, READS = MI + NI, GROUP = MI * NI;
    static_assert(READS <= GROUP && LOADS <= GROUP * KS, "the reads of a group and the loads of a tile fit behind the MFMAs");
    static_assert(((ROWS_PER_PASS >> SWZ) % KP) == 0 && ((32 >> SWZ) % KP) == 0,
                  "the swizzle term must repeat with the load pass and the 32-row MFMA block");

    __shared__ __attribute__((aligned(1024))) uint16_t Ps[STAGES][BM * BK];
    __shared__ __attribute__((aligned(1024))) uint16_t Qs[STAGES][BN * BK];

    // first_big < 0: the grid covers the tiles_m x tiles_n grid of BM x BN tiles. Otherwise this launch
    // finishes what a launch of a 256 x 256 kernel left over: tiles_m x tiles_n is that kernel's grid,
    // first_big the first tile number it did not take, and every leftover tile is cut into
    // (256 / BM) x (256 / BN) tiles of this kernel.
    int row0, col0;
    if (first_big < 0) {
        int tm, tn;
        xcd_tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn);
        row0 = tm * BM;
        col0 = tn * BN;
    } else {
        constexpr int SUB_M = 256 / BM, SUB_N = 256 / BN;
        int tm, tn;
        xcd_tile_coords(first_big + blockIdx.x / (SUB_M * SUB_N), tiles_m, tiles_n, tm, tn);
        const int sub = blockIdx.x % (SUB_M * SUB_N);
        row0 = tm * 256 + (sub / SUB_N) * BM;
        col0 = tn * 256 + (sub % SUB_N) * BN;
    }

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;
    const int l32 = lane & 31, lhi = lane >> 5;

    f32x16 acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    // Load side: lane l of a wave-wide load owns row l / KP of its rows and slot l % KP.
    const int ld_row = wave * ROWS_PER_LOAD + lane / KP;
    const int ld_chunk = (lane % KP) ^ ((ld_row >> SWZ) & (KP - 1));
    const uint32_t lane_off = (static_cast<uint32_t>(lane / KP) * static_cast<uint32_t>(ld) + ld_chunk * 8) * 2u;  // bytes
    const char* p_wave = reinterpret_cast<const char*>(P + static_cast<size_t>(row0 + wave * ROWS_PER_LOAD) * ld);
    const char* q_wave = reinterpret_cast<const char*>(Q + static_cast<size_t>(col0 + wave * ROWS_PER_LOAD) * ld);

    const size_t pass_bytes = static_cast<size_t>(ROWS_PER_PASS) * ld * 2;
    // Load number m (0 .. LOADS - 1) of the tile that starts at k0, into stage `stage`.
    const int p_first = row0 + wave * ROWS_PER_LOAD, q_first = col0 + wave * ROWS_PER_LOAD;
    const long long p_left = static_cast<long long>(R - p_first) * ld * 2, q_left = static_cast<long long>(Cn - q_first) * ld * 2;
    const i32x4 p_rsrc = buffer_descriptor(EDGE && p_left > 0 ? static_cast<const void*>(p_wave) : static_cast<const void*>(P), EDGE ? clamped_extent(p_left) : 0u);
    const i32x4 q_rsrc = buffer_descriptor(EDGE && q_left > 0 ? static_cast<const void*>(q_wave) : static_cast<const void*>(Q), EDGE ? clamped_extent(q_left) : 0u);
    const int k_full = K - K % BK;
    const uint32_t tail_off = (k_full + ld_chunk * 8 < K) ? lane_off : kBeyondExtent;
    auto issue_load = [&](int stage, int k0, int m) {
        if constexpr (EDGE) {
            const uint32_t off = k0 < k_full ? lane_off : (k0 < K ? tail_off : kBeyondExtent);
            if (m < P_PER)
                direct_load16_buffer(p_rsrc, off, static_cast<uint32_t>(k0) * 2u + m * static_cast<uint32_t>(pass_bytes),
                                     &Ps[stage][(m * ROWS_PER_PASS + wave * ROWS_PER_LOAD) * BK]);
            else
                direct_load16_buffer(q_rsrc, off, static_cast<uint32_t>(k0) * 2u + (m - P_PER) * static_cast<uint32_t>(pass_bytes),
                                     &Qs[stage][((m - P_PER) * ROWS_PER_PASS + wave * ROWS_PER_LOAD) * BK]);
        } else {
            if (m < P_PER)
                direct_load16(p_wave + static_cast<size_t>(k0) * 2 + m * pass_bytes, lane_off,
                              &Ps[stage][(m * ROWS_PER_PASS + wave * ROWS_PER_LOAD) * BK]);
            else
                direct_load16(q_wave + static_cast<size_t>(k0) * 2 + (m - P_PER) * pass_bytes, lane_off,
                              &Qs[stage][((m - P_PER) * ROWS_PER_PASS + wave * ROWS_PER_LOAD) * BK]);
        }
    };

    // Operand side: row (wave tile origin + 32 i + l32), chunk 2 kk + lhi of the row.
    const int sw = (l32 >> SWZ) & (KP - 1);
    int p_off[KS], q_off[KS];
#pragma unroll
    for (int kk = 0; kk < KS; ++kk) {
        const int slot = (2 * kk + lhi) ^ sw;
        p_off[kk] = (wave_m * WM + l32) * BK + slot * 8;
        q_off[kk] = (wave_n * WN + l32) * BK + slot * 8;
    }
    bf16x8 fa[2][MI], fb[2][NI];
    // Read number r (0 .. READS - 1) of k-group kk of the tile in `stage`, into operand slot kk & 1.
    auto read_one = [&](int stage, int kk, int r) {
        if (r < MI)
            fa[kk & 1][r] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(&Ps[stage][p_off[kk] + r * 32 * BK]));
        else
            fb[kk & 1][r - MI] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(&Qs[stage][q_off[kk] + (r - MI) * 32 * BK]));
    };
    // The MFMAs of operand slot `slot`; `after(m)` is issued right behind the m-th.
    auto mfma_group = [&](int slot, auto after) {
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int j = 0; j < NI; ++j) {
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[slot][i], fb[slot][j], acc[i][j], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
                after(i * NI + j);
                __builtin_amdgcn_sched_barrier(0);
            }
    };

    // One phase = everything between two barriers. Entered right after the barrier
    // that says "tile t is complete in stage S and nobody reads the stage of tile t-1
    // any more", while operand slot 1 holds the last k-group of tile t-1. Group g of
    // the phase (g = 0 .. KS-1) issues the MFMAs of the k-group read one group earlier
    // (g = 0: the last one of tile t-1); behind its first READS MFMAs go the reads of
    // k-group g of tile t, and behind the MFMAs of group 0 also the direct loads of tile
    // t+AHEAD into the stage tile t-1 has left. Then: wait until at most the loads of the
    // younger tiles are in flight, barrier.
    auto phase = [&](auto stage_c, auto prefetch, int k_next) {
        constexpr int S = decltype(stage_c)::value;
#pragma unroll
        for (int g = 0; g < KS; ++g) {
            mfma_group((g + 1) & 1, [&](int m) {
                // Reads of k-group g behind the first MFMAs of every group; the loads of the next tile one
                // behind each MFMA from the start of the phase (with 16 MFMAs per group all of them fall
                // into the first group), so that every load has most of the phase to land (spreading them
                // over two groups was slower for long K, issuing two per MFMA too).
                if (m < READS) read_one(S, g, m);
                if constexpr (prefetch) {
                    if (g * GROUP + m < LOADS) issue_load((S + AHEAD) % STAGES, k_next, g * GROUP + m);
                }
            });
        }
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(prefetch ? (AHEAD - 1) * LOADS : 0, 0));
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");  // the compiler does not know that the loads write LDS: no read moves above the barrier
        __builtin_amdgcn_sched_barrier(0);
    };
    using yes = std::integral_constant<bool, true>;
    using no = std::integral_constant<bool, false>;
    using s0 = std::integral_constant<int, 0>;
    using s1 = std::integral_constant<int, 1>;
    using s2 = std::integral_constant<int, 2>;
    using s3 = std::integral_constant<int, 3>;

    // Slot 1 starts as zeros, so the "previous tile" MFMAs of the first phase add nothing.
#pragma unroll
    for (int i = 0; i < MI; ++i) fa[1][i] = bf16x8{};
#pragma unroll
    for (int j = 0; j < NI; ++j) fb[1][j] = bf16x8{};

    // The launcher guarantees K % BK == 0 and at least STAGES tiles. Tile t lives in
    // stage (first + t) % STAGES with `first` chosen such that the last tile sits in the
    // last stage: the ragged part of the tile count is handled up front and the rest
    // runs in whole rings.
    const int k_tiles = EDGE ? ((K + BK - 1) / BK < STAGES ? STAGES : (K + BK - 1) / BK) : K / BK;
    const int ragged = k_tiles % STAGES;
    const int first = (STAGES - ragged) % STAGES;
#pragma unroll
    for (int t = 0; t < AHEAD; ++t)
#pragma unroll
        for (int m = 0; m < LOADS; ++m) issue_load((first + t) % STAGES, t * BK, m);
    __builtin_amdgcn_s_waitcnt(waitcnt_imm((AHEAD - 1) * LOADS, 0));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);

    int k_next = AHEAD * BK;  // first k of the tile the next phase prefetches
    if constexpr (STAGES == 4) {
        if (ragged == 3) { phase(s1{}, yes{}, k_next); k_next += BK; }
        if (ragged >= 2) { phase(s2{}, yes{}, k_next); k_next += BK; }
        if (ragged >= 1) { phase(s3{}, yes{}, k_next); k_next += BK; }
        for (int ring = k_tiles / STAGES; ring > 1; --ring) {
            phase(s0{}, yes{}, k_next);
            phase(s1{}, yes{}, k_next + BK);
            phase(s2{}, yes{}, k_next + 2 * BK);
            phase(s3{}, yes{}, k_next + 3 * BK);
            k_next += 4 * BK;
        }
        phase(s0{}, yes{}, k_next);
        phase(s1{}, no{}, 0);
        phase(s2{}, no{}, 0);
        phase(s3{}, no{}, 0);
    } else {
        if (ragged == 1) { phase(s1{}, yes{}, k_next); k_next += BK; }
        for (int ring = k_tiles / STAGES; ring > 1; --ring) {
            phase(s0{}, yes{}, k_next);
            phase(s1{}, yes{}, k_next + BK);
            k_next += 2 * BK;
        }
        phase(s0{}, yes{}, k_next);
        phase(s1{}, no{}, 0);
    }
    mfma_group(1, [](int) {});  // last k-group of the last tile

    if constexpr (RAGGED) {
        // The k values the loop left out are added on the way out (the product of two bf16 values is exact in
        // fp32): a lane holds 16 rows per 32-row block and one column per 32-column block.
        float qt[NI][7];
#pragma unroll
        for (int j = 0; j < NI; ++j) load_k_tail(Q, ld, col0, Cn, col0 + wave_n * WN + j * 32 + l32, K, K_all, qt[j]);
#pragma unroll
        for (int i = 0; i < MI; ++i) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = row0 + wave_m * WM + i * 32 + 8 * (v / 4) + 4 * lhi + (v % 4);
                float pt[7];
                load_k_tail(P, ld, row0, R, row, K, K_all, pt);
#pragma unroll
                for (int j = 0; j < NI; ++j) {
                    const int col = col0 + wave_n * WN + j * 32 + l32;
                    float r = acc[i][j][v];
#pragma unroll
                    for (int t = 0; t < 7; ++t) r = __builtin_fmaf(pt[t], qt[j][t], r);
                    if (row < R && col < Cn) store_out(&OUT[static_cast<size_t>(row) * Cn + col], r);
                }
            }
        }
        return;
    }
#pragma unroll
    for (int i = 0; i < MI; ++i) {
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            const int col = col0 + wave_n * WN + j * 32 + l32;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = row0 + wave_m * WM + i * 32 + 8 * (v / 4) + 4 * lhi + (v % 4);
                if (!EDGE || (row < R && col < Cn))
                    store_out(&OUT[static_cast<size_t>(row) * Cn + col], acc[i][j][v]);
            }
        }
    }
}

// ------------------------------------------- the 16x16x32 matrix instruction in place --
// v_mfma_f32_16x16x32_bf16: OUT (16 x 16) += P fragment (16 rows x 32 k) * Q fragment (16 rows x 32 k)^T;
// lane l supplies 8 consecutive k of row l % 16, starting at k = 8 (l / 16); result register v of lane l is
// OUT[4 (l / 16) + v][l % 16]. A wave's 128 x 128 tile is 8 x 8 such sub-tiles (64 accumulators of 4
// registers). Against v_mfma_f32_32x32x16_bf16 the instruction has the same peak rate and draws about
// 12 % less power per flop (register-only loops on random operands: 2.04 against 1.82 PFLOP/s).
//
// It is issued from inline assembly with the accumulator as a read-write operand: written with the
// builtin, the compiler gave result and addend different registers, and with all 256 accumulation
// registers taken by the 64 accumulators that meant moving them around in every iteration (hundreds of
// copies and spills). The compiler does not know the instruction's result latency then. What every site
// that uses it has to guarantee: (1) no instruction other than another in-place matrix instruction on the
// same accumulator reads or copies an accumulator within 64 idle cycles of the last instruction that wrote
// it: the only such place is the write-back, which calls mfma_results_settle() first; (2) a fragment
// register written by a vector instruction (not by an LDS read, whose wait the compiler inserts) is not
// used by the next five instructions: loops that start with a matrix instruction begin with five wait
// states; (3) all phases of a K loop are the same straight-line code inside one loop, so that the compiler
// has no reason to move accumulators between registers behind an instruction whose latency it cannot see.
__device__ __forceinline__ void mfma_16x16x32_in_place(f32x4& c, bf16x8 a, bf16x8 b) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}
__device__ __forceinline__ void mfma_results_settle() {
    asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory");
}

// ------------------------------ direct-to-LDS loads with early fragment reads, 16x16x32 --
// Whole tiles, an even number (at least 4) of K tiles. Global data goes straight into LDS (direct_load.h) as
// in the ring kernel, whose problem is that a stage has to be free before the load into it can be issued,
// which leaves a load less than one tile time (a pipeline that staged tiles through registers instead bought
// its lead time with 16 LDS write instructions per wave and K tile and was 2-3 % slower). Here all 32 fragments of a K
// tile are read into registers behind the first 32 matrix instructions of its phase (three sets of
// 8 + 8 fragments: k-step 0 of this tile, k-step 1 of this tile, k-step 1 of the previous tile, which is
// what those instructions multiply), a barrier in mid-phase then says that nobody reads the stage any
// more, and the loads of the tile after next are issued into it right away: about one and a half tile
// times before they are needed.
//
// RAGGED (with EDGE): K need not be a multiple of 8 and P, Q need only be 2 B aligned. The 16 B loads then
// start at 2 B-aligned addresses, which the memory path accepts (measured on gfx950, for the lane offset and
// for the descriptor's base). The K loop covers K rounded down to a multiple of 8, where every chunk lies
// inside its row, and the last K % 8 values of k are added in front of the write-back from ordinary loads.
//
// PERSIST (whole tiles only): a workgroup takes tiles blockIdx.x, blockIdx.x + gridDim.x, ... of n_tiles one after
// the other. The sixteen loads every phase issues, which in the last two phases of a tile have nothing left to
// fetch, then fetch the first two K tiles of the workgroup's NEXT tile: the next tile starts with its operands in
// LDS, the write-back's stores drain while it multiplies, and no workgroup is launched or retired in between.
template <int BM, int BN, int WM, int WN, bool EDGE, typename OutT, bool RAGGED = false, bool PERSIST = false>
__global__ __launch_bounds__((BM / WM) * (BN / WN) * kWave) void gemm_bf16_early_kernel(
    int R, int Cn, int K_all, const uint16_t* __restrict__ P, const uint16_t* __restrict__ Q,
    OutT* __restrict__ OUT, int tiles_m, int tiles_n, int n_tiles = 0) {
    static_assert(EDGE || !RAGGED, "the ragged form is an edge form");
    static_assert(!PERSIST || !EDGE, "the persistent form takes whole tiles");
    // ld: elements between rows of P and of Q. K: the part of the k range the loop covers.
    const int ld = K_all;
    const int K = RAGGED ? K_all - K_all % 8 : K_all;
    constexpr int BK = 64, KP = 8, SWZ = 1;
    constexpr int WAVES_N = BN / WN;
    constexpr int WAVES = (BM / WM) * WAVES_N;
    constexpr int MI = WM / 16, NI = WN / 16;
    static_assert(MI == 8 && NI == 8, "written for 128 x 128 wave tiles");
    constexpr int ROWS_PER_LOAD = kWave / KP;
    constexpr int ROWS_PER_PASS = ROWS_PER_LOAD * WAVES;
    constexpr int P_PER = BM / ROWS_PER_PASS, Q_PER = BN / ROWS_PER_PASS;
    constexpr int LOADS = P_PER + Q_PER;
    static_assert(LOADS == 16, "sixteen direct loads per wave and K tile");

    __shared__ __attribute__((aligned(1024))) uint16_t Ps[2][BM * BK];
    __shared__ __attribute__((aligned(1024))) uint16_t Qs[2][BN * BK];
    // Whole tiles: 16 rows x WN columns of bf16, or x WN / 2 columns of fp32, per wave on their way out (see
    // write_back_rows below).
    constexpr bool ROWS_OUT = !EDGE;
    constexpr int OUT_LD = WN + 8;  // 272 B rows: the sixteen lanes of a 16-row column of packets hit 16 different bank pairs
    __shared__ __attribute__((aligned(16))) uint16_t Out_s[ROWS_OUT ? WAVES : 1][ROWS_OUT ? 16 * OUT_LD : 8];
    int tile = blockIdx.x;
    int tm, tn;
    xcd_tile_coords(tile, tiles_m, tiles_n, tm, tn);
    int row0 = tm * BM, col0 = tn * BN;

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
    const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;
    const int l16 = lane & 15, lq = lane >> 4;

    f32x4 acc[MI][NI];

    // Load side, as in gemm_bf16_ring_kernel.
    const int ld_row = wave * ROWS_PER_LOAD + lane / KP;
    const int ld_chunk = (lane % KP) ^ ((ld_row >> SWZ) & (KP - 1));
    const uint32_t lane_off = (static_cast<uint32_t>(lane / KP) * static_cast<uint32_t>(ld) + ld_chunk * 8) * 2u;

    // The loads go through two buffer descriptors (this wave's first P row, its first Q row) for their
    // addressing mode, not for range checks: descriptor base + scalar offset + lane offset, where the scalar
    // offset (load number x rows per pass) and the lane offset are loop-invariant and only the two bases
    // move along K. With one 64-bit scalar base per load instead, the compiler keeps 32 pointers as
    // induction variables: some 90 scalar additions and a dozen reloads of spilled scalar registers in one
    // run at the head of every iteration, with the matrix pipe idle behind them.
    //
    // EDGE: R, Cn, K need not be whole tiles (K a multiple of 8, operands 16 B aligned). Then the range check
    // is used as well: the descriptors' extents end with the matrices, so rows beyond them arrive as zeros
    // (a descriptor whose base moves up by some bytes loses as many from its extent); what follows a row's
    // last column is the next row, so in the partial K tile lanes with k >= K use an offset beyond any
    // extent, and in the K tiles that pad the count to an even number of at least 4 all lanes do.
    // (Forced into a scalar register here: direct_load16_buffer_to_destination takes its scalar operands as
    // they are, so that no v_readfirstlane ends up right in front of a load.)
    const uint32_t pass_bytes = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(ROWS_PER_PASS) * static_cast<uint32_t>(ld) * 2u);  // the launcher keeps BM * K * 2 below 2^31
    // The two descriptors of the tile whose first row / column is r0 / c0.
    auto descriptors_of = [&](int r0, int c0, i32x4& p_desc, i32x4& q_desc) {
        const char* p_wave = reinterpret_cast<const char*>(P + static_cast<size_t>(r0 + wave * ROWS_PER_LOAD) * ld);
        const char* q_wave = reinterpret_cast<const char*>(Q + static_cast<size_t>(c0 + wave * ROWS_PER_LOAD) * ld);
        const int p_first = r0 + wave * ROWS_PER_LOAD, q_first = c0 + wave * ROWS_PER_LOAD;
        const long long p_left = static_cast<long long>(R - p_first) * ld * 2, q_left = static_cast<long long>(Cn - q_first) * ld * 2;
        p_desc = buffer_descriptor(EDGE && p_left <= 0 ? reinterpret_cast<const char*>(P) : p_wave, EDGE ? clamped_extent(p_left) : 0x7fffffffu);
        q_desc = buffer_descriptor(EDGE && q_left <= 0 ? reinterpret_cast<const char*>(Q) : q_wave, EDGE ? clamped_extent(q_left) : 0x7fffffffu);
    };
    i32x4 p_rsrc, q_rsrc;
    descriptors_of(row0, col0, p_rsrc, q_rsrc);
    auto advanced = [](i32x4 d, uint32_t bytes) {  // the descriptor with its base moved up
        const uint64_t a = ((static_cast<uint64_t>(static_cast<uint32_t>(d[1])) << 32) | static_cast<uint32_t>(d[0])) + bytes;
        d[0] = static_cast<int>(a & 0xffffffffu);
        d[1] = static_cast<int>(a >> 32);
        if constexpr (EDGE) {
            // Signed subtract and maximum (extents stay below 2^31), which the scalar ALU has: written as an
            // unsigned saturating subtraction this becomes a vector instruction plus v_readfirstlane, and
            // a scalar register written by the vector ALU is not safe to read in the load's inline assembly
            // a few cycles later (the compiler does not insert the wait states there).
            const int rest = d[2] - static_cast<int>(bytes);
            d[2] = rest > 0 ? rest : 0;
        }
        return d;
    };
    const int k_full = K - K % BK;
    const uint32_t tail_off = (k_full + ld_chunk * 8 < K) ? lane_off : kBeyondExtent;
    auto lane_offset_at = [&](int k0) -> uint32_t {  // k0 wave-uniform: the select costs one vector instruction per K tile
        if constexpr (!EDGE) return lane_off;
        return k0 < k_full ? lane_off : (k0 < K ? tail_off : kBeyondExtent);
    };
    // The two parts of a load in the K loop: the LDS destination goes into M0 one matrix instruction
    // before the load is issued (see set_direct_load_destination).
    auto aim_load = [&](int stage, int m) {
        set_direct_load_destination(m < P_PER ? &Ps[stage][(m * ROWS_PER_PASS + wave * ROWS_PER_LOAD) * BK]
                                              : &Qs[stage][((m - P_PER) * ROWS_PER_PASS + wave * ROWS_PER_LOAD) * BK]);
    };
    auto fire_load = [&](const i32x4& pd, const i32x4& qd, uint32_t off, int m) {
        if (m < P_PER) direct_load16_buffer_to_destination(pd, off, m * pass_bytes);
        else direct_load16_buffer_to_destination(qd, off, (m - P_PER) * pass_bytes);
    };
    auto issue_load = [&](int stage, const i32x4& pd, const i32x4& qd, uint32_t off, int m) {
        if (m < P_PER)
            direct_load16_buffer(pd, off, m * pass_bytes, &Ps[stage][(m * ROWS_PER_PASS + wave * ROWS_PER_LOAD) * BK]);
        else
            direct_load16_buffer(qd, off, (m - P_PER) * pass_bytes,
                                 &Qs[stage][((m - P_PER) * ROWS_PER_PASS + wave * ROWS_PER_LOAD) * BK]);
    };

    // Operand side.
    const int sw = (l16 >> SWZ) & (KP - 1);
    int p_off[2], q_off[2];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
        const int slot = (4 * kk + lq) ^ sw;
        p_off[kk] = (wave_m * WM + l16) * BK + slot * 8;
        q_off[kk] = (wave_n * WN + l16) * BK + slot * 8;
    }
    // Fragment sets: [0] k-step 0 of the current tile; [1], [2] k-step 1 of the tiles in stage 0 / stage 1.
    bf16x8 fp[3][MI], fq[3][NI];
    auto read_fragment = [&](int set, int stage, int kk, int r) {  // r = 0..7: P fragment r; 8..15: Q fragment r - 8
        if (r < MI)
            fp[set][r] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(&Ps[stage][p_off[kk] + r * 16 * BK]));
        else
            fq[set][r - MI] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(&Qs[stage][q_off[kk] + (r - MI) * 16 * BK]));
    };
    // The 64 instructions of one k-step from fragment set `set`; `after(m)` is issued right behind the m-th.
    // The sub-tiles are walked row by row, every other row backwards, so that consecutive instructions always
    // share one operand (measured 0.5-1 % over always walking forwards).
    auto mfma_block = [&](int set, auto after) {
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int jj = 0; jj < NI; ++jj) {
                const int j = (i & 1) ? NI - 1 - jj : jj;
                mfma_16x16x32_in_place(acc[i][j], fq[set][j], fp[set][i]);  // Q first: see the write-back
                __builtin_amdgcn_sched_barrier(0);
                after(i * NI + jj);
                __builtin_amdgcn_sched_barrier(0);
            }
    };

    // One phase, for the tile in stage S (tile t). Entered right after the barrier that says "tile t is
    // complete in stage S".
    //   k-step 1 of tile t-1 (set 2 - S... the set of the other stage); behind its first 32 instructions the
    //     32 fragment reads of tile t: k-step 0 into set 0, k-step 1 into the set of stage S
    //   wait for those reads; barrier: nobody reads stage S any more
    //   k-step 0 of tile t (set 0); behind its first instructions the direct loads of tile t+2 into stage S
    //   wait until at most those loads are in flight (tile t+1 has landed); barrier
    // Every phase issues its sixteen loads, the last two as well (they fetch the last two tiles once
    // more, into stages nobody reads again): all phases are then the same straight-line code inside one
    // loop, and the compiler keeps every accumulator in one place for the whole K loop. (With separate
    // code for the last two phases it moved accumulators between registers right behind matrix
    // instructions whose latency it does not know, see mfma_16x16x32_in_place, and read them too early;
    // with the loads under a run-time condition the branches cost 5 %.)
    auto phase = [&](auto stage_c, const i32x4& p_from, const i32x4& q_from, uint32_t k_next_bytes, bool wait_at_end) {
        constexpr int S = decltype(stage_c)::value;
        constexpr int MINE = 1 + S, OTHER = 2 - S;  // fragment sets of k-step 1: this stage's, the other stage's
        // Load number n goes behind instruction BARRIER_AT + n * GAP of the phase's 128 (counted from the
        // start of the first block); the barrier that frees the stage sits behind instruction BARRIER_AT - 1.
        constexpr int BARRIER_AT = kEarlyBarrierAt, GAP = kEarlyLoadGap;
        static_assert(BARRIER_AT >= 33 && BARRIER_AT <= 64 && BARRIER_AT + (LOADS - 1) * GAP < 128, "loads fit the phase");
        const i32x4 pd = advanced(p_from, k_next_bytes), qd = advanced(q_from, k_next_bytes);
        const uint32_t off = lane_offset_at(static_cast<int>(k_next_bytes / 2));
        auto maybe_load = [&](int at) {  // `at` = number of the instruction just issued, 0..127
            if (at + 1 >= BARRIER_AT && (at + 1 - BARRIER_AT) % GAP == 0 && (at + 1 - BARRIER_AT) / GAP < LOADS)
                aim_load(S, (at + 1 - BARRIER_AT) / GAP);
            if (at >= BARRIER_AT && (at - BARRIER_AT) % GAP == 0 && (at - BARRIER_AT) / GAP < LOADS)
                fire_load(pd, qd, off, (at - BARRIER_AT) / GAP);
        };
        mfma_block(OTHER, [&](int m) {
            if (m < 16) read_fragment(0, S, 0, m);
            else if (m < 32) read_fragment(MINE, S, 1, m - 16);
            if (m == BARRIER_AT - 1) {
                __builtin_amdgcn_s_waitcnt(waitcnt_imm(kVmMax, 0));
                __builtin_amdgcn_s_barrier();
                __builtin_amdgcn_sched_barrier(0);
            }
            maybe_load(m);
        });
        mfma_block(0, [&](int m) { maybe_load(64 + m); });
        if (wait_at_end) __builtin_amdgcn_s_waitcnt(waitcnt_imm(LOADS, kLgkmMax));
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");  // the compiler does not know that the loads write LDS: no read moves above the barrier
        __builtin_amdgcn_sched_barrier(0);
    };
    using s0 = std::integral_constant<int, 0>;
    using s1 = std::integral_constant<int, 1>;

    // Tile t lives in stage t % 2. Whole tiles: the launcher guarantees an even number of K tiles, at least 4;
    // EDGE: the count is padded to one (the padding tiles load zeros).
    const int k_tiles = EDGE ? (ceil_div(K, BK) < 4 ? 4 : (ceil_div(K, BK) + 1) / 2 * 2) : K / BK;
    // The workgroups of XCD x start their walk along K at tile k_first = x * stagger (even) and
    // wrap around, so that at any time the eight XCDs fetch from eight different column windows of the
    // operands instead of all 256 workgroups from the same 128 B of 8192 rows. (All workgroups of one XCD
    // keep the same phase: they share panels through its L2.)
    int k_first = 0;
    if constexpr (kEarlyKStagger != 0) {
        const int step = kEarlyKStagger;
        k_first = __builtin_amdgcn_readfirstlane((static_cast<int>(blockIdx.x % kXcds) * step) % k_tiles);
    }
    auto k_bytes_of = [&](int t) -> uint32_t {  // byte offset along K of the t-th tile of this workgroup's walk
        const int at = t + k_first;
        return static_cast<uint32_t>(at < k_tiles ? at : at - k_tiles) * (BK * 2);
    };
    {
        const i32x4 pd = advanced(p_rsrc, k_bytes_of(0)), qd = advanced(q_rsrc, k_bytes_of(0));
        const uint32_t off = lane_offset_at(static_cast<int>(k_bytes_of(0) / 2));
#pragma unroll
        for (int m = 0; m < LOADS; ++m) issue_load(0, pd, qd, off, m);
    }
    {
        const i32x4 pd = advanced(p_rsrc, k_bytes_of(1)), qd = advanced(q_rsrc, k_bytes_of(1));
        const uint32_t off = lane_offset_at(static_cast<int>(k_bytes_of(1) / 2));
#pragma unroll
        for (int m = 0; m < LOADS; ++m) issue_load(1, pd, qd, off, m);
    }
    // PERSIST: both K tiles have landed at the head of every tile (see the wait in front of the write-back).
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(PERSIST ? 0 : LOADS, kLgkmMax));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
  while (true) {   // one output tile per trip (a single trip unless PERSIST)
    // Entered with the tile's first K tile complete in stage 0 and its second one on the way into stage 1.
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j) acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    // "k-step 1 of the tile before the first" multiplies zeros (set 2 is what the first phase, stage 0, uses).
#pragma unroll
    for (int i = 0; i < MI; ++i) fp[2][i] = bf16x8{};
#pragma unroll
    for (int j = 0; j < NI; ++j) fq[2][j] = bf16x8{};
    // The workgroup's next tile, if it has one: what the last two phases fetch.
    const int next_tile = PERSIST ? tile + static_cast<int>(gridDim.x) : 0;
    const bool has_next = PERSIST && next_tile < n_tiles;
    int next_row0 = row0, next_col0 = col0;
    i32x4 p_next = p_rsrc, q_next = q_rsrc;
    if (has_next) {
        xcd_tile_coords(next_tile, tiles_m, tiles_n, tm, tn);
        next_row0 = tm * BM;
        next_col0 = tn * BN;
        descriptors_of(next_row0, next_col0, p_next, q_next);
    }
    for (int t = 0; t < k_tiles; t += 2) {
        // Fragment registers that the vector ALU has written (the zeros of set 2 above, and the copies the
        // compiler makes of them in front of the loop) need wait states before a matrix instruction reads
        // them. The compiler inserts those for its own matrix instructions, not for one in inline assembly:
        // in a variant of this loop that began right at a matrix instruction, the first one read stale
        // registers on some lanes (0 x NaN from whatever ran before = NaN in the first sub-tile, on the first
        // call only). Here scalar instructions happen to sit in between; the five wait states make that
        // independent of what the compiler puts at the head of the loop, and cost nothing measurable.
        asm volatile("s_nop 4");
        // What this pair of phases fetches: K tiles t + 2 and t + 3 of this tile; in the last trip the first two K
        // tiles of the next tile, or, without one, the last two of this tile once more. Selected, not branched
        // on: the trips stay the same straight-line code.
        const bool last = t + 2 >= k_tiles;
        const int next = last ? (has_next ? 0 : k_tiles - 2) : t + 2;
        const uint32_t k_next_bytes = k_bytes_of(next);  // k_first and next are even: next + 1 does not wrap
        i32x4 p_from = p_rsrc, q_from = q_rsrc;
        if (last) {
            p_from = p_next;
            q_from = q_next;
        }
        // PERSIST: the first phase of a tile does not wait at its end. What that wait is for, the tile's second K
        // tile, has landed already, and the loads are counted in order: it would wait for the 64 stores of the
        // tile before, which sit in front of this phase's loads. They get one more phase to drain.
        phase(s0{}, p_from, q_from, k_next_bytes, !PERSIST || t != 0);
        phase(s1{}, p_from, q_from, k_next_bytes + BK * 2, true);
    }
    // k-step 1 of the last tile (stage 1 -> set 2). Outside the loop the compiler is free to move accumulators
    // to other registers; it does so between these instructions, so here they are issued through the builtin,
    // whose result latency it knows.
    mfma_results_settle();
    // Every later use of an accumulator takes it from here, behind the wait states: without this the compiler is
    // free to copy accumulators in front of them (they are no memory operation, which is all the settling
    // assembly orders), and in the persistent form it did.
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j) asm volatile("" : "+a"(acc[i][j]));
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fq[2][j], fp[2][i], acc[i][j], 0, 0, 0);
    // Write-back. The matrix instructions are given the Q fragment first, i.e. they form the transposed
    // sub-tile (Q rows) x (P rows): register v of lane l then holds OUT[row l % 16][column 4 (l / 16) + v] of
    // the sub-tile, four consecutive columns, and a lane stores them as one packet (16 B of fp32, 8 B of bf16)
    // instead of four separate elements. Tiles that lie wholly inside the matrix (all of them unless EDGE)
    // store without guards; rows need only be aligned like their elements.
    auto store_packet = [&](OutT* at, const f32x4& r) {
        if constexpr (std::is_same<OutT, float>::value) {
            typedef float f32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
            *reinterpret_cast<f32x4_a4*>(at) = r;
        } else {
            typedef uint16_t u16x4_a2 __attribute__((ext_vector_type(4), aligned(2)));
            *reinterpret_cast<u16x4_a2*>(at) = u16x4_a2{f32_to_bf16_rne(r[0]), f32_to_bf16_rne(r[1]), f32_to_bf16_rne(r[2]), f32_to_bf16_rne(r[3])};
        }
    };
    auto write_back = [&](auto guarded) {
#pragma unroll
        for (int i = 0; i < MI; ++i) {
            const int row = row0 + wave_m * WM + i * 16 + l16;
#pragma unroll
            for (int j = 0; j < NI; ++j) {
                const int col = col0 + wave_n * WN + j * 16 + 4 * lq;
                OutT* at = &OUT[static_cast<size_t>(row) * Cn + col];
                if constexpr (!guarded) {
                    store_packet(at, acc[i][j]);
                } else {  // tiles that hang over an edge: element by element
#pragma unroll
                    for (int v = 0; v < 4; ++v)
                        if (row < R && col + v < Cn) store_out(at + v, acc[i][j][v]);
                }
            }
        }
    };
    // Whole tiles: a lane's packet of four results is 8 B of bf16 or 16 B of fp32, and its neighbours' packets lie in
    // other rows (lane l holds row l % 16), so one store instruction would be 64 separate writes, which cost the memory
    // pipeline as much as 64 wider ones: in a store-only loop 8 us per bf16 tile and CU against 2.3 us for the same
    // bytes written as 256 B runs (fp32, with output that stays in L2: 7.2 against 4.6). So 16 rows at a time go through
    // LDS: packets in (a wave's own patch of 16 rows x 256 B, rows padded by 16 B), rows out, 16 B per lane, sixteen
    // lanes to a row, four rows to a store. LDS executes a wave's accesses in order: no waits between the two.
    // fp32 gains 1-3 % (16384 x 16384 x 1024: 14 %): a round's 67 MB from all CUs at once are bound by the write
    // bandwidth whatever the pattern. bf16, together with the hardware's conversion: 17-30 % at K up to 1024.
    auto write_back_rows = [&]() {
        if constexpr (ROWS_OUT && std::is_same<OutT, float>::value) {
            typedef float f32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
            char* mine = reinterpret_cast<char*>(Out_s[wave]);
#pragma unroll
            for (int i = 0; i < MI; ++i) {
#pragma unroll
                for (int jh = 0; jh < 2; ++jh) {
#pragma unroll
                    for (int jj = 0; jj < 4; ++jj)
                        *reinterpret_cast<f32x4*>(mine + l16 * (OUT_LD * 2) + jj * 64 + lq * 16) = acc[i][4 * jh + jj];
#pragma unroll
                    for (int p = 0; p < 4; ++p) {
                        const int in_block = 4 * p + lq;
                        const f32x4 v = *reinterpret_cast<const f32x4*>(mine + in_block * (OUT_LD * 2) + 16 * l16);
                        const int row = row0 + wave_m * WM + i * 16 + in_block;
                        const int col = col0 + wave_n * WN + jh * 64 + 4 * l16;
                        *reinterpret_cast<f32x4_a4*>(&OUT[static_cast<size_t>(row) * Cn + col]) = v;
                    }
                }
            }
        } else if constexpr (ROWS_OUT) {
            typedef uint16_t u16x4 __attribute__((ext_vector_type(4)));
            typedef uint32_t u32x4_a2 __attribute__((ext_vector_type(4), aligned(2)));
            uint16_t* mine = Out_s[wave];
#pragma unroll
            for (int i = 0; i < MI; ++i) {
#pragma unroll
                for (int j = 0; j < NI; ++j) {
                    const f32x4& r = acc[i][j];
                    *reinterpret_cast<u16x4*>(mine + l16 * OUT_LD + j * 16 + 4 * lq) =
                        u16x4{f32_to_bf16_rne(r[0]), f32_to_bf16_rne(r[1]), f32_to_bf16_rne(r[2]), f32_to_bf16_rne(r[3])};
                }
#pragma unroll
                for (int p = 0; p < 4; ++p) {
                    const int in_block = 4 * p + lq;  // lanes 16 q .. 16 q + 15 take row 4 p + q
                    const u32x4 v = *reinterpret_cast<const u32x4*>(mine + in_block * OUT_LD + 8 * l16);
                    const int row = row0 + wave_m * WM + i * 16 + in_block;
                    const int col = col0 + wave_n * WN + 8 * l16;
                    *reinterpret_cast<u32x4_a2*>(&OUT[static_cast<size_t>(row) * Cn + col]) = u32x4_a2{v[0], v[1], v[2], v[3]};
                }
            }
        }
    };
    if constexpr (RAGGED) {
        // The k values the loop left out (K_all % 8 of them, at most 7) are added on the way out (load_k_tail
        // above): a lane holds 8 rows x 32 columns (four consecutive ones per sub-tile). The product of two bf16
        // values is exact in fp32.
        float pt[MI][7];
#pragma unroll
        for (int i = 0; i < MI; ++i) load_k_tail(P, ld, row0, R, row0 + wave_m * WM + i * 16 + l16, K, K_all, pt[i]);
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            const int col = col0 + wave_n * WN + j * 16 + 4 * lq;
            float qt[4][7];
#pragma unroll
            for (int v = 0; v < 4; ++v) load_k_tail(Q, ld, col0, Cn, col + v, K, K_all, qt[v]);
#pragma unroll
            for (int i = 0; i < MI; ++i) {
                const int row = row0 + wave_m * WM + i * 16 + l16;
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    float r = acc[i][j][v];
#pragma unroll
                    for (int t = 0; t < 7; ++t) r = __builtin_fmaf(pt[i][t], qt[v][t], r);
                    if (row < R && col + v < Cn) store_out(&OUT[static_cast<size_t>(row) * Cn + col + v], r);
                }
            }
            __builtin_amdgcn_sched_barrier(0);  // one column block at a time: its 28 Q values and no more
        }
    } else {
        // PERSIST: the next tile's first two K tiles (fetched by the last two phases) land before the stores queue up
        // behind them; its first phase relies on that.
        if constexpr (PERSIST) __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, kLgkmMax));
        if constexpr (ROWS_OUT) write_back_rows();
        else if (!EDGE || (row0 + BM <= R && col0 + BN <= Cn)) write_back(std::false_type{});
        else write_back(std::true_type{});
    }
    if (!has_next) break;
    tile = next_tile;
    row0 = next_row0;
    col0 = next_col0;
    p_rsrc = p_next;
    q_rsrc = q_next;
  }
    // The last, redundant loads write LDS: they must have landed before the wave ends and its LDS goes to
    // the next workgroup. Behind the write-back the wait is covered by the stores.
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, kLgkmMax));
}

// Up to 16 rows of one operand against all rows of the other: D[f][g] = sum_k F[f][k] * G[g][k], f < f_count <= 16.
// The strips that a matrix leaves beyond whole 256 x 256 tiles when it hangs over them by a few rows or columns go
// here instead of into a round of edge tiles of their own (4097 x 4097 x 4096: one round of whole tiles plus two
// strips instead of 289 guarded tiles in two rounds). Reading G bounds it: one 16 x 16 x 32 matrix instruction per 1 KB
// of G, both fragments straight from global memory (F stays in the caches). A workgroup takes 16 rows of G; its eight
// waves split K and add their parts in a fixed order. K is a multiple of 8 and both operands are 16 B aligned.
// ALONG_G: OUT[f * ldo + g] (extra rows of P: F = those rows, G = Q); else OUT[g * ldo + f] (extra rows of Q, i.e.
// extra columns of OUT: F = those rows, G = P). The instruction gets the operand first whose index runs along OUT's
// rows, so that a lane's four results are neighbours in memory (see the write-back of gemm_bf16_early_kernel).
constexpr int kThinMax = 16, kThinWaves = 8;
template <bool ALONG_G, typename OutT>
__global__ __launch_bounds__(kThinWaves * kWave) void gemm_bf16_thin_kernel(
    int f_count, int g_count, int K, const uint16_t* __restrict__ F, const uint16_t* __restrict__ G,
    OutT* __restrict__ OUT, long long ldo) {
    __shared__ f32x4 part[kThinWaves][kWave];
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    const int l16 = lane % 16, lq = lane / 16;
    const int g0 = static_cast<int>(blockIdx.x) * 16;
    const bool f_ok = l16 < f_count, g_ok = g0 + l16 < g_count;
    const uint16_t* f_at = F + static_cast<size_t>(f_ok ? l16 : 0) * K + 8 * lq;
    const uint16_t* g_at = G + static_cast<size_t>(g_ok ? g0 + l16 : 0) * K + 8 * lq;
    // Steps of 32 along K; wave w takes steps [w * per, (w + 1) * per). The last step may be short: packets of
    // 8 that begin at or beyond K are zeros.
    const int steps = ceil_div(K, 32), per = ceil_div(steps, kThinWaves);
    const int first = wave * per, last = first + per < steps ? first + per : steps;
    constexpr int U = 4;
    f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int step = first; step < last; step += U) {
        bf16x8 fv[U], gv[U];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int k = (step + u) * 32;
            const bool in = step + u < last && k + 8 * lq < K;
            fv[u] = in && f_ok ? *reinterpret_cast<const bf16x8*>(f_at + k) : bf16x8{};
            gv[u] = in && g_ok ? *reinterpret_cast<const bf16x8*>(g_at + k) : bf16x8{};
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
            acc = ALONG_G ? __builtin_amdgcn_mfma_f32_16x16x32_bf16(gv[u], fv[u], acc, 0, 0, 0)
                          : __builtin_amdgcn_mfma_f32_16x16x32_bf16(fv[u], gv[u], acc, 0, 0, 0);
    }
    part[wave][lane] = acc;
    __syncthreads();
    if (wave != 0) return;
    f32x4 sum = part[0][lane];
#pragma unroll
    for (int w = 1; w < kThinWaves; ++w) sum += part[w][lane];
    // ALONG_G: the lane holds D[f = l16][g = g0 + 4 lq + v]; else D[f = 4 lq + v][g = g0 + l16].
#pragma unroll
    for (int v = 0; v < 4; ++v) {
        const int f = ALONG_G ? l16 : 4 * lq + v, g = ALONG_G ? g0 + 4 * lq + v : g0 + l16;
        if (f < f_count && g < g_count)
            store_out(&OUT[ALONG_G ? f * ldo + g : g * ldo + f], sum[v]);
    }
}

// Whole 256 x 256 tiles with K a multiple of 128, at least 384: tiles_m x tiles_n of them from the top left corner
// of OUT (R and Cn bound the operands and give OUT's row length; they may reach beyond the tiles).
template <int BM, int BN, int WM, int WN, typename OutT>
int run_whole_tiles(int R, int Cn, int K, const uint16_t* P, const uint16_t* Q, OutT* OUT, int tiles_m, int tiles_n,
                    hipStream_t s) {
    const dim3 block((BM / WM) * (BN / WN) * kWave);

    // Tile counts that do not fill whole rounds of CUs: the 256 x 256 kernel takes the whole rounds and
    // the tiles of the last, partial round are cut into 128 x 128 tiles (two workgroups per CU), when
    // that gives every CU at most two of them (6144^3: 2 rounds + 64 tiles instead of 3 rounds).
    static_assert(BM == 256 && BN == 256, "the leftover launch cuts 256 x 256 tiles");
    const int tiles = tiles_m * tiles_n, cus = cu_count();
    const int left = tiles % cus;
    const bool cut = tiles > cus && left != 0 && left * 4 <= 2 * cus;
    const int main_tiles = cut ? tiles - left : tiles;
    if (main_tiles > cus && cus % 8 == 0)   // more than one round: one workgroup per CU walks its tiles (see PERSIST)
        gemm_bf16_early_kernel<BM, BN, WM, WN, false, OutT, false, true><<<dim3(static_cast<unsigned>(cus)), block, 0, s>>>(
            R, Cn, K, P, Q, OUT, tiles_m, tiles_n, main_tiles);
    else
        gemm_bf16_early_kernel<BM, BN, WM, WN, false, OutT><<<dim3(static_cast<unsigned>(main_tiles)), block, 0, s>>>(
            R, Cn, K, P, Q, OUT, tiles_m, tiles_n);
    if (int rc = check_launch("gemm_bf16_early_kernel")) return rc;
    if (cut) {
        if (left * 4 <= cus)  // one per CU: the four-deep ring, as below
            gemm_bf16_ring_kernel<128, 128, 64, 4, 64, 64, false, OutT><<<dim3(static_cast<unsigned>(left) * 4), dim3(256), 0, s>>>(
                R, Cn, K, P, Q, OUT, tiles_m, tiles_n, main_tiles);
        else
            gemm_bf16_ring_kernel<128, 128, 64, 2, 64, 64, false, OutT><<<dim3(static_cast<unsigned>(left) * 4), dim3(256), 0, s>>>(
                R, Cn, K, P, Q, OUT, tiles_m, tiles_n, main_tiles);
        return check_launch("gemm_bf16_ring_kernel (leftover)");
    }
    return 0;
}

// Kernel choice. Whole 256 x 256 x 64 tiles: the early-read pipeline whenever the K tile count is even and
// at least 6, else the direct-to-LDS ring (any count from 2). Ragged M, N or K with K a multiple of 8 and
// 16 B-aligned operands: the early-read pipeline's edge variant (K tiles padded with zeros to an even count).
// Rows that are not 16 B aligned: its ragged form. At most 128 tiles: 128 x 128 tiles of the ring, with the
// same edge and ragged forms. Everything else: the general kernel.
template <int BM, int BN, int BK, int WM, int WN, typename OutT>
int run_gemm_bf16(int R, int Cn, int K, const uint16_t* P, const uint16_t* Q, OutT* OUT,
                  hipStream_t s) {
    constexpr int LD = BK + 8;
    constexpr size_t lds_bytes = 2ull * (BM + BN) * LD * sizeof(uint16_t);
    const int tiles_m = ceil_div(R, BM), tiles_n = ceil_div(Cn, BN);
    const dim3 grid(static_cast<unsigned>(tiles_m) * tiles_n), block((BM / WM) * (BN / WN) * kWave);
    const bool aligned = aligned16(P) && aligned16(Q);
    const bool whole = (R % BM == 0) && (Cn % BN == 0) && aligned;
    // A 256-row panel (plus up to six K tiles of padding) is addressed with 32-bit offsets.
    const bool panel_ok = static_cast<long long>(BM > BN ? BM : BN) * (static_cast<long long>(K) + 6 * 64) * 2 < (1ll << 31);
    // Up to half as many 256 x 256 tiles as CUs: as 128 x 128 tiles they still all run at once, two to a CU
    // (1024 x 8192 x 8192, 128 tiles: 1050 -> 1190 TFLOP/s; with more tiles the small ones lose, 160: 1170 -> 900).
    const bool few_tiles = static_cast<long long>(tiles_m) * tiles_n * 2 <= cu_count();
    const bool lane_offsets_ok = static_cast<long long>(K) * 2 * 64 < (1ll << 32);  // 32-bit lane offsets inside a load's rows
    // A few rows or columns beyond whole tiles (at most kThinMax each way) over at least half a round of whole
    // tiles: the whole tiles as below, the rest as strips (gemm_bf16_thin_kernel).
    const int r_thin = R % BM, c_thin = Cn % BN;
    if ((r_thin != 0 || c_thin != 0) && r_thin <= kThinMax && c_thin <= kThinMax && aligned && K % 128 == 0 && K >= 6 * 64 &&
        panel_ok && lane_offsets_ok && static_cast<long long>(R / BM) * (Cn / BN) * 2 >= cu_count()) {
        const int Rw = R - r_thin, Cw = Cn - c_thin;
        if (int rc = run_whole_tiles<BM, BN, WM, WN, OutT>(R, Cn, K, P, Q, OUT, Rw / BM, Cw / BN, s)) return rc;
        const dim3 thin_block(kThinWaves * kWave);
        if (r_thin != 0) {  // rows Rw.. of OUT, all columns
            gemm_bf16_thin_kernel<true, OutT><<<dim3(static_cast<unsigned>(ceil_div(Cn, 16))), thin_block, 0, s>>>(
                r_thin, Cn, K, P + static_cast<size_t>(Rw) * K, Q, OUT + static_cast<size_t>(Rw) * Cn, Cn);
            if (int rc = check_launch("gemm_bf16_thin_kernel (rows)")) return rc;
        }
        if (c_thin != 0) {  // columns Cw.. of OUT, the rows of the whole tiles
            gemm_bf16_thin_kernel<false, OutT><<<dim3(static_cast<unsigned>(ceil_div(Rw, 16))), thin_block, 0, s>>>(
                c_thin, Rw, K, Q + static_cast<size_t>(Cw) * K, P, OUT + Cw, Cn);
            if (int rc = check_launch("gemm_bf16_thin_kernel (columns)")) return rc;
        }
        return 0;
    }
    if (whole && !few_tiles && K % 128 == 0 && K >= 6 * 64 && panel_ok && lane_offsets_ok)
        return run_whole_tiles<BM, BN, WM, WN, OutT>(R, Cn, K, P, Q, OUT, tiles_m, tiles_n, s);
    // The same for rows that are not 16 B aligned (K not a multiple of 8, operands at an odd element).
    if (few_tiles && !(aligned && K % 8 == 0) && K >= 8 && panel_ok) {
        const int tm = ceil_div(R, 128), tn = ceil_div(Cn, 128);
        const dim3 grid128(static_cast<unsigned>(tm) * tn);
        if (K >= 256 && tm * tn <= cu_count())
            gemm_bf16_ring_kernel<128, 128, 64, 4, 64, 64, true, OutT, true><<<grid128, dim3(256), 0, s>>>(R, Cn, K, P, Q, OUT, tm, tn, -1);
        else
            gemm_bf16_ring_kernel<128, 128, 64, 2, 64, 64, true, OutT, true><<<grid128, dim3(256), 0, s>>>(R, Cn, K, P, Q, OUT, tm, tn, -1);
        return check_launch("gemm_bf16_ring_kernel (128 x 128, ragged rows)");
    }
    // Too few 256 x 256 tiles for the CUs: 128 x 128 tiles (four waves of 64 x 64), two workgroups per CU.
    if (few_tiles && aligned && K % 8 == 0 && K > 0 && panel_ok) {
        const int tm = ceil_div(R, 128), tn = ceil_div(Cn, 128);
        const dim3 grid128(static_cast<unsigned>(tm) * tn);
        const bool whole128 = R % 128 == 0 && Cn % 128 == 0 && K % 64 == 0;
        // At most one workgroup per CU: nothing else hides the memory latency, so the ring is four K tiles
        // deep (128 KB of LDS) instead of two.
        if (whole128 && K >= 256 && tm * tn <= cu_count())
            gemm_bf16_ring_kernel<128, 128, 64, 4, 64, 64, false, OutT><<<grid128, dim3(256), 0, s>>>(R, Cn, K, P, Q, OUT, tm, tn, -1);
        else if (whole128 && K >= 128)
            gemm_bf16_ring_kernel<128, 128, 64, 2, 64, 64, false, OutT><<<grid128, dim3(256), 0, s>>>(R, Cn, K, P, Q, OUT, tm, tn, -1);
        else if (K >= 256 && tm * tn <= cu_count())
            gemm_bf16_ring_kernel<128, 128, 64, 4, 64, 64, true, OutT><<<grid128, dim3(256), 0, s>>>(R, Cn, K, P, Q, OUT, tm, tn, -1);
        else
            gemm_bf16_ring_kernel<128, 128, 64, 2, 64, 64, true, OutT><<<grid128, dim3(256), 0, s>>>(R, Cn, K, P, Q, OUT, tm, tn, -1);
        return check_launch("gemm_bf16_ring_kernel (128 x 128)");
    }
    if (whole && K % 64 == 0 && K >= 64 * 2 && lane_offsets_ok) {
        gemm_bf16_ring_kernel<BM, BN, 64, 2, WM, WN, false, OutT>
            <<<grid, block, 0, s>>>(R, Cn, K, P, Q, OUT, tiles_m, tiles_n, -1);
        return check_launch("gemm_bf16_ring_kernel");
    }
    // The edge forms of the early-read kernel. As with whole tiles, the tiles of a partial last round (at most half
    // the CUs' worth) are cut into 128 x 128 tiles of the ring, two workgroups per CU (8190^3: 1089 tiles, 4 rounds
    // and 65 tiles cut into 260 instead of 5 rounds).
    auto edge_tiles = [&](auto ragged, const char* what) -> int {
        constexpr bool RG = decltype(ragged)::value;
        const int tiles = tiles_m * tiles_n, cus = cu_count();
        const int left = tiles % cus;
        const bool cut = tiles > cus && left != 0 && left * 4 <= 2 * cus;
        const int main_tiles = cut ? tiles - left : tiles;
        gemm_bf16_early_kernel<BM, BN, WM, WN, true, OutT, RG><<<dim3(static_cast<unsigned>(main_tiles)), block, 0, s>>>(
            R, Cn, K, P, Q, OUT, tiles_m, tiles_n);
        if (int rc = check_launch(what)) return rc;
        if (cut) {
            if (left * 4 <= cus && K >= 256)
                gemm_bf16_ring_kernel<128, 128, 64, 4, 64, 64, true, OutT, RG><<<dim3(static_cast<unsigned>(left) * 4), dim3(256), 0, s>>>(
                    R, Cn, K, P, Q, OUT, tiles_m, tiles_n, main_tiles);
            else
                gemm_bf16_ring_kernel<128, 128, 64, 2, 64, 64, true, OutT, RG><<<dim3(static_cast<unsigned>(left) * 4), dim3(256), 0, s>>>(
                    R, Cn, K, P, Q, OUT, tiles_m, tiles_n, main_tiles);
            return check_launch("gemm_bf16_ring_kernel (leftover, edges)");
        }
        return 0;
    };
    // Ragged M, N or K with 16 B-aligned rows: the early-read kernel with zero-filled edges.
    if (aligned && K % 8 == 0 && K > 0 && panel_ok && lane_offsets_ok)
        return edge_tiles(std::false_type{}, "gemm_bf16_early_kernel (edges)");
    // Rows that are not 16 B aligned (K not a multiple of 8, or operands at an odd element): its ragged form,
    // when there are enough tiles for the CUs and at least one group of 8 along K.
    if (!few_tiles && K >= 8 && panel_ok && lane_offsets_ok)
        return edge_tiles(std::true_type{}, "gemm_bf16_early_kernel (ragged rows)");
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(gemm_bf16_kernel<BM, BN, BK, WM, WN, true, OutT>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(lds_bytes));
    if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(gemm_bf16_kernel)");
    gemm_bf16_kernel<BM, BN, BK, WM, WN, true, OutT><<<grid, block, lds_bytes, s>>>(R, Cn, K, P, Q, OUT, tiles_m, tiles_n);
    return check_launch("gemm_bf16_kernel");
}

}  // namespace

int launch_gemm_bf16(int M, int N, int K, const uint16_t* A, const uint16_t* B, float* D_f32,
                     uint16_t* C_bf16_colmajor, hipStream_t s) {
    if (M < 0 || N < 0 || K < 0) return fail(1, "prism_gemm_bf16: negative dimension (%d,%d,%d)", M, N, K);
    if (M == 0 || N == 0) return 0;
    if ((D_f32 == nullptr) == (C_bf16_colmajor == nullptr))
        return fail(1, "prism_gemm_bf16: exactly one output must be given");
    if (K > 0 && (A == nullptr || B == nullptr)) return fail(1, "prism_gemm_bf16: null matrix pointer");
    if (!aligned2(A) || !aligned2(B) || !aligned4(D_f32) || !aligned2(C_bf16_colmajor))
        return fail(1, "prism_gemm_bf16: misaligned pointer");
    if (D_f32) return run_gemm_bf16<256, 256, 64, 128, 128, float>(M, N, K, A, B, D_f32, s);
    // Column-major M x N == row-major N x M of B @ A^T.
    return run_gemm_bf16<256, 256, 64, 128, 128, uint16_t>(N, M, K, B, A, C_bf16_colmajor, s);
}

}  // namespace prism
