// bf16 x bf16 -> fp32-accumulate GEMM on MFMA: OUT[r][c] = sum_k P[r][k] * Q[c][k],
// P is R x K and Q is Cn x K, both row-major bf16 (K contiguous), OUT row-major.
//
// This is the gfx950 counterpart of the reference's Hopper kernel
// (examples/h100_matmul.py:20-297, generated/cutlass_my_h100_match_no_tail.cu):
//   reference                                   here
//   wgmma m64n256k16 from swizzled smem     ->  v_mfma_f32_32x32x16_bf16 from padded LDS rows
//   TMA bulk copies + mbarrier ring (4 x)   ->  16 B global loads staged in registers one K
//                                               step ahead, two LDS buffers, one barrier a step
//   1 producer + 2 consumer warpgroups      ->  every wave loads and multiplies
//   persistent CTAs + 16x8 super-tiles      ->  one workgroup per tile, XCD-aware tile order
//   K tail dropped, M/N multiples required  ->  any M, N, K (zero-filled edge tiles)
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
// LDS rows are BK + 8 elements (144 B for BK = 64): eight lanes reading 16 B from
// eight consecutive rows then cover all banks exactly once.
#include <type_traits>

#include "common.h"
#include "tile_map.h"

// Block tile BM x BN x BK and wave tile WM x WN.
#ifndef PRISM_BF16_SCHED
#define PRISM_BF16_SCHED 1
#endif
#ifndef PRISM_BF16_DMA
#define PRISM_BF16_DMA 1
#endif
#ifndef PRISM_BF16_CFG
#define PRISM_BF16_CFG 256, 256, 64, 128, 128
#endif

namespace prism {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

// fp32 -> bf16, round to nearest even; NaN stays NaN (quiet bit forced).
__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) {
    const uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((u >> 16) | 0x0040u);
    return static_cast<uint16_t>((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
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
            uint16_t e[8];
#pragma unroll
            for (int c = 0; c < 8; ++c)
                e[c] = (row < rows && k + c < K) ? base[static_cast<size_t>(row) * K + k + c] : uint16_t{0};
            u32x4 r;
#pragma unroll
            for (int c = 0; c < 4; ++c) r[c] = static_cast<uint32_t>(e[2 * c]) | (static_cast<uint32_t>(e[2 * c + 1]) << 16);
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
#if PRISM_BF16_SCHED
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
#endif
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

// ------------------------------------------------------- full-tile kernel --
// Same product for problems made of whole tiles with 16 B aligned rows; global
// data goes straight into LDS (global_load_lds_dwordx4, no staging registers,
// no LDS-write instructions), which is the role TMA plays in the reference
// (evals/h100_bench/utils.cuh:238-273).
//
// A wave-wide direct load writes 1 KiB of contiguous LDS (lane l lands at
// base + 16 l), so rows cannot be padded. Bank conflicts are avoided the way the
// reference's 128 B swizzle does it (utils.cuh:6-16): the 16 B chunk c of row r
// is stored in slot c ^ ((r >> SWZ) & (chunks_per_row - 1)); the load side
// applies the permutation to the global address, the MFMA operand reads apply it
// to the LDS address.
//
// Two LDS stages of one K tile each, declared as separate arrays so that the
// compiler's wait-count logic knows loads into one stage do not feed reads of
// the other. Step t: issue the loads of tile t+1 into the idle stage, multiply
// tile t, barrier (which also waits for the loads), prefetch the first operands
// of tile t+1.
#ifndef PRISM_BF16_DMA_SPLIT
#define PRISM_BF16_DMA_SPLIT 1
#endif
#ifndef PRISM_BF16_SWZ
#define PRISM_BF16_SWZ 1
#endif

template <int BM, int BN, int BK, int WM, int WN, int SWZ, typename OutT>
__global__ __launch_bounds__((BM / WM) * (BN / WN) * kWave) void gemm_bf16_dma_kernel(
    int R, int Cn, int K, const uint16_t* __restrict__ P, const uint16_t* __restrict__ Q,
    OutT* __restrict__ OUT, int tiles_m, int tiles_n) {
    constexpr int WAVES_N = BN / WN;
    constexpr int WAVES = (BM / WM) * WAVES_N;
    constexpr int MI = WM / 32, NI = WN / 32;
    constexpr int KP = BK / 8;                       // 16 B chunks per row
    constexpr int KS = BK / 16;                      // k-substeps per tile
    constexpr int ROWS_PER_LOAD = kWave / KP;        // rows one wave-wide load covers
    constexpr int ROWS_PER_PASS = ROWS_PER_LOAD * WAVES;
    static_assert(BM % ROWS_PER_PASS == 0 && BN % ROWS_PER_PASS == 0, "whole load passes");
    constexpr int P_PER = BM / ROWS_PER_PASS, Q_PER = BN / ROWS_PER_PASS;  // loads per wave per tile
    static_assert(KS % 2 == 0 && (KP & (KP - 1)) == 0, "tile shape");
    static_assert(((ROWS_PER_PASS >> SWZ) % KP) == 0 && ((32 >> SWZ) % KP == 0 || KP <= (32 >> SWZ)),
                  "the swizzle term must repeat with the load pass and the 32-row MFMA block");

    __shared__ __attribute__((aligned(1024))) uint16_t Ps0[BM * BK];
    __shared__ __attribute__((aligned(1024))) uint16_t Ps1[BM * BK];
    __shared__ __attribute__((aligned(1024))) uint16_t Qs0[BN * BK];
    __shared__ __attribute__((aligned(1024))) uint16_t Qs1[BN * BK];

    int tm, tn;
    xcd_tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn);
    const int row0 = tm * BM, col0 = tn * BN;

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);  // wave-uniform, lives in an SGPR
    const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;
    const int l32 = lane & 31, lhi = lane >> 5;

    f32x16 acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    // Load side: in pass u this wave fills LDS rows [u * ROWS_PER_PASS + wave * ROWS_PER_LOAD, + ROWS_PER_LOAD);
    // lane l owns row (l / KP) of those and slot (l % KP), which holds global chunk
    // slot ^ swizzle(row). The swizzle term is the same in every pass, so the lane's
    // byte offset from the pass's first row is loop-invariant and everything else is scalar.
    const int ld_row = wave * ROWS_PER_LOAD + lane / KP;
    const int ld_chunk = (lane % KP) ^ ((ld_row >> SWZ) & (KP - 1));
    const uint32_t lane_off = static_cast<uint32_t>((lane / KP) * K + ld_chunk * 8) * 2u;  // bytes
    const char* p_wave = reinterpret_cast<const char*>(P + static_cast<size_t>(row0 + wave * ROWS_PER_LOAD) * K);
    const char* q_wave = reinterpret_cast<const char*>(Q + static_cast<size_t>(col0 + wave * ROWS_PER_LOAD) * K);
    const size_t pass_bytes = static_cast<size_t>(ROWS_PER_PASS) * K * 2;

    typedef const __attribute__((address_space(1))) void* gptr_t;
    typedef __attribute__((address_space(3))) void* lptr_t;
    auto issue_loads = [&](uint16_t* ps, uint16_t* qs, int k0) {
#pragma unroll
        for (int u = 0; u < P_PER; ++u)
            __builtin_amdgcn_global_load_lds((gptr_t)(p_wave + u * pass_bytes + static_cast<size_t>(k0) * 2 + lane_off),
                                             (lptr_t)(ps + (u * ROWS_PER_PASS + wave * ROWS_PER_LOAD) * BK), 16, 0, 0);
#pragma unroll
        for (int u = 0; u < Q_PER; ++u)
            __builtin_amdgcn_global_load_lds((gptr_t)(q_wave + u * pass_bytes + static_cast<size_t>(k0) * 2 + lane_off),
                                             (lptr_t)(qs + (u * ROWS_PER_PASS + wave * ROWS_PER_LOAD) * BK), 16, 0, 0);
    };

    // Operand side: row (wave tile origin + 32 i + l32), chunk (2 kk + lhi) -> slot.
    const int sw = (l32 >> SWZ) & (KP - 1);
    int p_off[KS], q_off[KS];  // element offsets inside a stage for i = 0 / j = 0
#pragma unroll
    for (int kk = 0; kk < KS; ++kk) {
        const int slot = (2 * kk + lhi) ^ sw;
        p_off[kk] = (wave_m * WM + l32) * BK + slot * 8;
        q_off[kk] = (wave_n * WN + l32) * BK + slot * 8;
    }
    bf16x8 fa[2][MI], fb[2][NI];
    auto read_frags = [&](const uint16_t* ps, const uint16_t* qs, int kk, int slot) {
#pragma unroll
        for (int i = 0; i < MI; ++i)
            fa[slot][i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(&ps[p_off[kk] + i * 32 * BK]));
#pragma unroll
        for (int j = 0; j < NI; ++j)
            fb[slot][j] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(&qs[q_off[kk] + j * 32 * BK]));
    };

    auto mfma_all = [&](int slot) {
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int j = 0; j < NI; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[slot][i], fb[slot][j], acc[i][j], 0, 0, 0);
    };

    // One phase = everything between two barriers. It is entered right after the
    // barrier that says "tile t is complete in (ps, qs), nobody reads (ps_n, qs_n)
    // any more", and while operand slot 1 still holds the last k-substep of tile
    // t-1. That substep's MFMAs are issued here, after the barrier, so that they
    // cover the barrier skew and the latency of the first operand reads of tile t:
    //   read substep 0 of tile t          -> slot 0
    //   MFMAs of the last substep of t-1  <- slot 1, with the direct loads of tile t+1 issued between them
    //   substeps 0 .. KS-2 of tile t, each preceded by the reads of the next substep
    //   barrier (also waits for the direct loads)
    // `prefetch`: tile t+1 exists and goes to (ps_n, qs_n).
    auto phase = [&](uint16_t* ps, uint16_t* qs, uint16_t* ps_n, uint16_t* qs_n, int k_next, auto prefetch) {
        read_frags(ps, qs, 0, 0);
        mfma_all(1);
        if constexpr (prefetch) issue_loads(ps_n, qs_n, k_next);
#pragma unroll
        for (int kk = 0; kk + 1 < KS; ++kk) {
            read_frags(ps, qs, kk + 1, (kk + 1) & 1);
            mfma_all(kk & 1);
        }
#if PRISM_BF16_SCHED
        // The direct loads are spread over the first DMA_SPLIT groups of MFMAs.
        constexpr int LOADS = prefetch ? (P_PER + Q_PER) : 0;
        constexpr int L_PER = (LOADS + PRISM_BF16_DMA_SPLIT - 1) / PRISM_BF16_DMA_SPLIT;
        __builtin_amdgcn_sched_group_barrier(0x100, MI + NI, 0);
        sched_substep<0, 0, L_PER, MI * NI>();
#pragma unroll
        for (int kk = 0; kk + 1 < KS; ++kk) {
            if (kk + 1 < PRISM_BF16_DMA_SPLIT)
                sched_substep<MI + NI, 0, L_PER, MI * NI>();
            else
                sched_substep<MI + NI, 0, 0, MI * NI>();
        }
#endif
        __syncthreads();
    };
    using yes = std::integral_constant<bool, true>;
    using no = std::integral_constant<bool, false>;

    // Slot 1 starts as zeros, so the "previous tile" MFMAs of the first phase add nothing.
#pragma unroll
    for (int i = 0; i < MI; ++i) fa[1][i] = bf16x8{};
#pragma unroll
    for (int j = 0; j < NI; ++j) fb[1][j] = bf16x8{};

    // The launcher guarantees K % BK == 0 and K > 0. Tiles alternate between the
    // two stages such that the last tile always sits in stage 1.
    const int k_tiles = K / BK;
    int t = 0;
    if (k_tiles & 1) {
        issue_loads(Ps1, Qs1, 0);
        __syncthreads();
        if (k_tiles > 1) {
            phase(Ps1, Qs1, Ps0, Qs0, BK, yes{});
            t = 1;
        }
    } else {
        issue_loads(Ps0, Qs0, 0);
        __syncthreads();
    }
    for (; t + 2 < k_tiles; t += 2) {
        phase(Ps0, Qs0, Ps1, Qs1, (t + 1) * BK, yes{});
        phase(Ps1, Qs1, Ps0, Qs0, (t + 2) * BK, yes{});
    }
    if (k_tiles > 1) phase(Ps0, Qs0, Ps1, Qs1, (t + 1) * BK, yes{});
    phase(Ps1, Qs1, Ps0, Qs0, 0, no{});
    mfma_all(1);  // last k-substep of the last tile

#pragma unroll
    for (int i = 0; i < MI; ++i) {
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            const int col = col0 + wave_n * WN + j * 32 + l32;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = row0 + wave_m * WM + i * 32 + 8 * (v / 4) + 4 * lhi + (v % 4);
                store_out(&OUT[static_cast<size_t>(row) * Cn + col], acc[i][j][v]);
            }
        }
    }
}

template <int BM, int BN, int BK, int WM, int WN, typename OutT>
int run_gemm_bf16(int R, int Cn, int K, const uint16_t* P, const uint16_t* Q, OutT* OUT,
                  hipStream_t s) {
    constexpr int LD = BK + 8;
    constexpr size_t lds_bytes = 2ull * (BM + BN) * LD * sizeof(uint16_t);
    const int tiles_m = ceil_div(R, BM), tiles_n = ceil_div(Cn, BN);
    const dim3 grid(static_cast<unsigned>(tiles_m) * tiles_n), block((BM / WM) * (BN / WN) * kWave);
    const bool fast = (K > 0) && (R % BM == 0) && (Cn % BN == 0) && (K % BK == 0) && aligned16(P) && aligned16(Q);
    auto launch = [&](auto kernel) -> int {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize,
                                           static_cast<int>(lds_bytes));
        if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute(gemm_bf16_kernel)");
        kernel<<<grid, block, lds_bytes, s>>>(R, Cn, K, P, Q, OUT, tiles_m, tiles_n);
        return check_launch("gemm_bf16_kernel");
    };
    if (fast) {
#if PRISM_BF16_DMA
        gemm_bf16_dma_kernel<BM, BN, BK, WM, WN, PRISM_BF16_SWZ, OutT><<<grid, block, 0, s>>>(R, Cn, K, P, Q, OUT, tiles_m, tiles_n);
        return check_launch("gemm_bf16_dma_kernel");
#else
        return launch(gemm_bf16_kernel<BM, BN, BK, WM, WN, false, OutT>);
#endif
    }
    return launch(gemm_bf16_kernel<BM, BN, BK, WM, WN, true, OutT>);
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
    if (D_f32) return run_gemm_bf16<PRISM_BF16_CFG, float>(M, N, K, A, B, D_f32, s);
    // Column-major M x N == row-major N x M of B @ A^T.
    return run_gemm_bf16<PRISM_BF16_CFG, uint16_t>(N, M, K, B, A, C_bf16_colmajor, s);
}

}  // namespace prism
