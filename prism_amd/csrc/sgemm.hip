// fp32 SGEMM progression, C = alpha * A @ B + beta * C, row-major, gfx950.
//
// The six kernels follow the reference's progression one to one
// (launch shapes: evals/4090_sgemm/runner.cu:135-243):
//   1  naive            generated/my_sgemm_kernel_1.cu       one thread per C element
//   2  coalesced        generated/my_sgemm_kernel_2.cu       32x32-tile thread remap
//   3  LDS block tile   generated/sgemm_shared_mem_block.cu  32x32 tiles in LDS
//   6  thread tile      generated/my_sgemm_kernel_3.cu       8x8 per thread, scalar staging
//   4  thread tile vec  generated/my_sgemm_kernel_4.cu       + 16 B loads, A tile transposed
//   5  wave tile        generated/my_sgemm_kernel_5.cu,
//                       evals/4090_sgemm/my_kernel_utils.cuh:13-90
// Kernels 1, 2, 3, 4 and 6 accumulate every C element with one fused
// multiply-add per k, in increasing k, and finish with
// fma(alpha, acc, beta * c): they are bit-identical to each other and to a
// serial host loop written the same way. Kernel 5 keeps the reference's
// block -> wave -> sub-tile decomposition, but a 64-lane wave computes its
// sub-tiles with v_mfma_f32_32x32x2_f32 instead of per-thread outer products;
// its summation order inside the matrix unit is not specified, so it is
// checked against an fp64 product within a tolerance. It comes in three forms,
// chosen by the launcher from the tile count: a direct-to-LDS kernel on
// 256 x 256 tiles for problems with enough such tiles to fill the chip (on
// 128 x 256 or 64 x 256 tiles below that, and for a partial last round), a
// one-wave-per-tile kernel for small problems and for some partial rounds, and
// the general 128 x 128 block kernel for shapes and alignments the others refuse.
// The two direct-to-LDS kernels have edge variants for ragged M, N, K with N and K
// multiples of 4 (16 B-aligned rows): their loads go through buffer descriptors
// whose range check zero-fills everything beyond the matrices. Both also have a
// form for rows that are only 4 B aligned (any N and K, matrices at any
// element). What is left (K < 4, offsets beyond 32 bits) takes the general
// kernel, whose edge variant uses range-checked 16 B buffer loads plus masks.
//
// Unlike the reference kernels (no guards in kernels 1, 3, 4, 5), every kernel
// here accepts any M, N, K. When beta == 0, C is not read.
#include <algorithm>

#include "common.h"
#include "direct_load.h"
#include "tile_map.h"

namespace prism {
namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float epilogue(float alpha, float acc, float beta, const float* c) {
    return beta == 0.0f ? alpha * acc : __builtin_fmaf(alpha, acc, beta * (*c));
}

// ---------------------------------------------------------------- kernel 1 --
// Thread id -> (row, col) = (tid / N, tid % N) as in
// generated/my_sgemm_kernel_1.cu:11-23, plus the bound the reference lacks.
__global__ __launch_bounds__(256) void sgemm_naive_kernel(int M, int N, int K, float alpha,
                                                          const float* __restrict__ A,
                                                          const float* __restrict__ B, float beta,
                                                          float* C) {
    const size_t tid = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (tid >= static_cast<size_t>(M) * N) return;
    const size_t row = tid / N, col = tid % N;
    float acc = 0.0f;
    for (int k = 0; k < K; ++k) acc = __builtin_fmaf(A[row * K + k], B[static_cast<size_t>(k) * N + col], acc);
    float* c = &C[row * N + col];
    *c = epilogue(alpha, acc, beta, c);
}

// ---------------------------------------------------------------- kernel 2 --
// Consecutive thread ids fill 32x32 tiles of C row by row
// (generated/my_sgemm_kernel_2.cu:5-16); block = one tile = 1024 threads.
__global__ __launch_bounds__(1024) void sgemm_coalesced_kernel(int M, int N, int K, float alpha,
                                                               const float* __restrict__ A,
                                                               const float* __restrict__ B,
                                                               float beta, float* C) {
    constexpr int TS = 32;
    const int tiles_per_row = (N + TS - 1) / TS;
    const int tile_row = blockIdx.x / tiles_per_row, tile_col = blockIdx.x % tiles_per_row;
    const int row = tile_row * TS + threadIdx.x / TS;
    const int col = tile_col * TS + threadIdx.x % TS;
    if (row >= M || col >= N) return;
    const float* a = A + static_cast<size_t>(row) * K;
    float acc = 0.0f;
    for (int k = 0; k < K; ++k) acc = __builtin_fmaf(a[k], B[static_cast<size_t>(k) * N + col], acc);
    float* c = &C[static_cast<size_t>(row) * N + col];
    *c = epilogue(alpha, acc, beta, c);
}

// ---------------------------------------------------------------- kernel 3 --
// 32x32 tiles of A and B staged in LDS, one accumulator per thread, two
// barriers per K tile exactly where the reference's sync pass puts them
// (generated/sgemm_shared_mem_block.cu:34,38). Out-of-range elements are
// staged as zeros. A wave reads one As word per row (broadcast) and 32
// consecutive Bs words, so neither tile needs padding.
__global__ __launch_bounds__(1024) void sgemm_lds_block_kernel(int M, int N, int K, float alpha,
                                                               const float* __restrict__ A,
                                                               const float* __restrict__ B,
                                                               float beta, float* C,
                                                               int num_blocks_n) {
    constexpr int BS = 32;
    __shared__ float As[BS * BS];
    __shared__ float Bs[BS * BS];
    const int c_row = blockIdx.x / num_blocks_n, c_col = blockIdx.x % num_blocks_n;
    const int t_row = threadIdx.x / BS, t_col = threadIdx.x % BS;
    const int row = c_row * BS + t_row, col = c_col * BS + t_col;
    float acc = 0.0f;
    for (int k0 = 0; k0 < K; k0 += BS) {
        const int ka = k0 + t_col, kb = k0 + t_row;
        As[t_row * BS + t_col] = (row < M && ka < K) ? A[static_cast<size_t>(row) * K + ka] : 0.0f;
        Bs[t_row * BS + t_col] = (kb < K && col < N) ? B[static_cast<size_t>(kb) * N + col] : 0.0f;
        __syncthreads();
        // Always the whole tile: the zero-filled tail adds exact +0 products, so
        // the result still equals the serial loop over k < K bit for bit.
#pragma unroll
        for (int d = 0; d < BS; ++d) acc = __builtin_fmaf(As[t_row * BS + d], Bs[d * BS + t_col], acc);
        __syncthreads();
    }
    if (row < M && col < N) {
        float* c = &C[static_cast<size_t>(row) * N + col];
        *c = epilogue(alpha, acc, beta, c);
    }
}

// ----------------------------------------------------------- kernels 4 / 6 --
// Block tile BM x BN, K step BK, TM x TN accumulators per thread.
//   VEC = false: kernel 6 (generated/my_sgemm_kernel_3.cu): A tile row-major
//                [BM][BK], scalar staging.
//   VEC = true : kernel 4 (generated/my_sgemm_kernel_4.cu:41-46,74-79): A tile
//                stored transposed [BK][BM], 16 B global loads, 16 B C epilogue.
//   EDGE       : predicated scalar staging and stores for tiles that hang over
//                M, N or K, or when rows are not 16 B aligned.
// The register-fill loops are bounded by TM for regM and TN for regN; the
// reference bounds both by TN (examples/sgemm_kernel_3.py:66-67), which is only
// right because TM == TN there.
template <int BM, int BN, int BK, int TM, int TN, bool VEC, bool EDGE>
__global__ __launch_bounds__((BM * BN) / (TM * TN)) void sgemm_thread_tile_kernel(
    int M, int N, int K, float alpha, const float* __restrict__ A, const float* __restrict__ B,
    float beta, float* C, int num_blocks_n) {
    constexpr int THREADS = (BM * BN) / (TM * TN);
    static_assert(TN % 4 == 0 && BK % 4 == 0 && BN % 4 == 0, "16 B packets");
    __shared__ __attribute__((aligned(16))) float As[BM * BK];
    __shared__ __attribute__((aligned(16))) float Bs[BK * BN];

    const int c_row = blockIdx.x / num_blocks_n, c_col = blockIdx.x % num_blocks_n;
    const int row0 = c_row * BM, col0 = c_col * BN;
    const int tid = threadIdx.x;
    const int t_row = tid / (BN / TN), t_col = tid % (BN / TN);

    float acc[TM * TN] = {0.0f};
    float reg_m[TM], reg_n[TN];

    for (int k0 = 0; k0 < K; k0 += BK) {
        if constexpr (VEC && !EDGE) {
            // 16 B packets: A along k, stored transposed; B along n, stored as is.
            for (int p = tid; p < BM * BK / 4; p += THREADS) {
                const int r = p / (BK / 4), kc = p % (BK / 4);
                const f32x4 a = *reinterpret_cast<const f32x4*>(
                    &A[static_cast<size_t>(row0 + r) * K + k0 + kc * 4]);
                As[(kc * 4 + 0) * BM + r] = a.x;
                As[(kc * 4 + 1) * BM + r] = a.y;
                As[(kc * 4 + 2) * BM + r] = a.z;
                As[(kc * 4 + 3) * BM + r] = a.w;
            }
            for (int p = tid; p < BK * BN / 4; p += THREADS) {
                const int r = p / (BN / 4), nc = p % (BN / 4);
                *reinterpret_cast<f32x4*>(&Bs[r * BN + nc * 4]) = *reinterpret_cast<const f32x4*>(
                    &B[static_cast<size_t>(k0 + r) * N + col0 + nc * 4]);
            }
        } else {
            for (int p = tid; p < BM * BK; p += THREADS) {
                const int r = p / BK, kk = p % BK;
                float a;
                if constexpr (EDGE)
                    a = (row0 + r < M && k0 + kk < K) ? A[static_cast<size_t>(row0 + r) * K + k0 + kk] : 0.0f;
                else
                    a = A[static_cast<size_t>(row0 + r) * K + k0 + kk];
                if constexpr (VEC) As[kk * BM + r] = a; else As[r * BK + kk] = a;
            }
            for (int p = tid; p < BK * BN; p += THREADS) {
                const int r = p / BN, nn = p % BN;
                float b;
                if constexpr (EDGE)
                    b = (k0 + r < K && col0 + nn < N) ? B[static_cast<size_t>(k0 + r) * N + col0 + nn] : 0.0f;
                else
                    b = B[static_cast<size_t>(k0 + r) * N + col0 + nn];
                Bs[r * BN + nn] = b;
            }
        }
        __syncthreads();
#pragma unroll
        for (int d = 0; d < BK; ++d) {
#pragma unroll
            for (int i = 0; i < TM; ++i)
                reg_m[i] = VEC ? As[d * BM + t_row * TM + i] : As[(t_row * TM + i) * BK + d];
#pragma unroll
            for (int j = 0; j < TN; ++j) reg_n[j] = Bs[d * BN + t_col * TN + j];
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i * TN + j] = __builtin_fmaf(reg_m[i], reg_n[j], acc[i * TN + j]);
        }
        __syncthreads();
    }

#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int row = row0 + t_row * TM + i;
        if constexpr (VEC && !EDGE) {
#pragma unroll
            for (int j = 0; j < TN; j += 4) {
                f32x4* c = reinterpret_cast<f32x4*>(&C[static_cast<size_t>(row) * N + col0 + t_col * TN + j]);
                f32x4 r;
                if (beta == 0.0f) {
                    r.x = alpha * acc[i * TN + j + 0];
                    r.y = alpha * acc[i * TN + j + 1];
                    r.z = alpha * acc[i * TN + j + 2];
                    r.w = alpha * acc[i * TN + j + 3];
                } else {
                    const f32x4 old = *c;
                    r.x = __builtin_fmaf(alpha, acc[i * TN + j + 0], beta * old.x);
                    r.y = __builtin_fmaf(alpha, acc[i * TN + j + 1], beta * old.y);
                    r.z = __builtin_fmaf(alpha, acc[i * TN + j + 2], beta * old.z);
                    r.w = __builtin_fmaf(alpha, acc[i * TN + j + 3], beta * old.w);
                }
                *c = r;
            }
        } else {
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int col = col0 + t_col * TN + j;
                if (!EDGE || (row < M && col < N)) {
                    float* c = &C[static_cast<size_t>(row) * N + col];
                    *c = epilogue(alpha, acc[i * TN + j], beta, c);
                }
            }
        }
    }
}

// ---------------------------------------------------------------- kernel 5 --
// Block tile BM x BN split over (BM/WM) x (BN/WN) waves; a wave's WM x WN tile
// is a grid of 32x32 sub-tiles (the WMITER x WNITER sub-tiles of
// generated/my_sgemm_kernel_5.cu:8-10 with WSUBM = WSUBN = 32), each held as the
// 16 accumulator registers of one v_mfma_f32_32x32x2_f32.
//
// LDS tiles (double-buffered, one barrier per K step):
//   As[k][m], transposed like the reference's loadFromGmem
//   (evals/4090_sgemm/my_kernel_utils.cuh:23-31): row length BM + 2 words so
//   that the four k-rows a 16 B global packet scatters to hit distinct banks;
//   Bs[k][n] as in global memory.
// MFMA operands: lane l supplies A[m = l % 32][k = l / 32] and
// B[k = l / 32][n = l % 32]: both are 32 consecutive LDS words per half-wave.
// Result register v of lane l is C[8 * (v / 4) + 4 * (l / 32) + v % 4][l % 32].
//
// Global loads for K step t+1 are issued before the MFMAs of step t and written
// to the other LDS buffer after them.
//
// Workgroups are dealt to the 8 XCDs round-robin by id; the id is remapped so
// that every XCD walks its own contiguous band of C tiles in columns of 8, and
// the tiles resident on one XCD share A and B panels in that XCD's L2.
template <int BM, int BN, int BK, int WM, int WN, bool EDGE>
__global__ __launch_bounds__((BM / WM) * (BN / WN) * kWave)
__attribute__((amdgpu_waves_per_eu(4))) void sgemm_wave_tile_kernel(
    int M, int N, int K, float alpha, const float* __restrict__ A, const float* __restrict__ B,
    float beta, float* C, int tiles_m, int tiles_n) {
    constexpr int WAVES_N = BN / WN;
    constexpr int THREADS = (BM / WM) * WAVES_N * kWave;
    constexpr int MI = WM / 32, NI = WN / 32;  // sub-tiles per wave
    constexpr int LDA = BM + 2, LDB = BN;
    constexpr int A_PACKETS = BM * BK / 4, B_PACKETS = BK * BN / 4;
    static_assert(A_PACKETS % THREADS == 0 && B_PACKETS % THREADS == 0, "whole packets per thread");
    constexpr int A_PER = A_PACKETS / THREADS, B_PER = B_PACKETS / THREADS;
    static_assert(BK % 4 == 0 && WM % 32 == 0 && WN % 32 == 0, "tile shapes");

    __shared__ __attribute__((aligned(16))) float As[2][BK * LDA];
    __shared__ __attribute__((aligned(16))) float Bs[2][BK * LDB];

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

    f32x4 a_stage[A_PER], b_stage[B_PER];

    // EDGE (any M, N, K; rows only 4 B aligned): 16 B buffer loads. The descriptor of A covers this
    // tile's row panel up to the end of the matrix and that of B is rebuilt per K tile from its first
    // row, so every dword at or beyond the end of a matrix (A rows >= M, B rows >= K) arrives as zero
    // from the range check and vector offsets stay small. What lies past the end of a row is the next
    // row: those elements (k >= K in A, columns >= N in B) are replaced by zeros after the load.
    auto clamp_extent = [](long long bytes) -> int {
        return static_cast<int>(bytes < 0 ? 0 : (bytes > 0x7fffffff ? 0x7fffffff : bytes));
    };
    const long long a_left = static_cast<long long>(M - row0) * K * 4;
    const auto a_rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<float*>(A + (a_left > 0 ? static_cast<size_t>(row0) * K : size_t{0})), 0, clamp_extent(a_left), 0x00020000);
    auto load_global = [&](int k0) {
#pragma unroll
        for (int u = 0; u < A_PER; ++u) {
            const int p = tid + u * THREADS;
            const int r = p / (BK / 4), kc = p % (BK / 4);
            const int row = row0 + r, k = k0 + kc * 4;
            if constexpr (!EDGE) {
                a_stage[u] = *reinterpret_cast<const f32x4*>(&A[static_cast<size_t>(row) * K + k]);
            } else {
                a_stage[u] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(
                    a_rsrc, (static_cast<uint32_t>(r) * static_cast<uint32_t>(K) + kc * 4) * 4u, k0 * 4, 0));
                if (k0 + BK > K) {
#pragma unroll
                    for (int c = 0; c < 4; ++c) a_stage[u][c] = (k + c < K) ? a_stage[u][c] : 0.0f;
                }
            }
        }
        const long long b_left = (static_cast<long long>(K - k0) * N - col0) * 4;
        const auto b_rsrc = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<float*>(B + (EDGE && b_left > 0 ? static_cast<size_t>(k0) * N + col0 : size_t{0})), 0,
            clamp_extent(b_left), 0x00020000);
#pragma unroll
        for (int u = 0; u < B_PER; ++u) {
            const int p = tid + u * THREADS;
            const int r = p / (BN / 4), nc = p % (BN / 4);
            const int k = k0 + r, col = col0 + nc * 4;
            if constexpr (!EDGE) {
                b_stage[u] = *reinterpret_cast<const f32x4*>(&B[static_cast<size_t>(k) * N + col]);
            } else {
                b_stage[u] = __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(
                    b_rsrc, (static_cast<uint32_t>(r) * static_cast<uint32_t>(N) + nc * 4) * 4u, 0, 0));
#pragma unroll
                for (int c = 0; c < 4; ++c) b_stage[u][c] = (col + c < N) ? b_stage[u][c] : 0.0f;
            }
        }
    };
    auto store_lds = [&](int buf) {
#pragma unroll
        for (int u = 0; u < A_PER; ++u) {
            const int p = tid + u * THREADS;
            const int r = p / (BK / 4), kc = p % (BK / 4);
#pragma unroll
            for (int c = 0; c < 4; ++c) As[buf][(kc * 4 + c) * LDA + r] = a_stage[u][c];
        }
#pragma unroll
        for (int u = 0; u < B_PER; ++u) {
            const int p = tid + u * THREADS;
            const int r = p / (BN / 4), nc = p % (BN / 4);
            *reinterpret_cast<f32x4*>(&Bs[buf][r * LDB + nc * 4]) = b_stage[u];
        }
    };

    const int k_tiles = (K + BK - 1) / BK;
    load_global(0);
    store_lds(0);
    __syncthreads();

    for (int t = 0; t < k_tiles; ++t) {
        const int buf = t & 1;
        const bool more = (t + 1 < k_tiles);
        if (more) load_global((t + 1) * BK);

        const float* as = &As[buf][wave_m * WM + l32];
        const float* bs = &Bs[buf][wave_n * WN + l32];
#pragma unroll
        for (int kk = 0; kk < BK; kk += 2) {
            float a[MI], b[NI];
#pragma unroll
            for (int i = 0; i < MI; ++i) a[i] = as[(kk + lhi) * LDA + i * 32];
#pragma unroll
            for (int j = 0; j < NI; ++j) b[j] = bs[(kk + lhi) * LDB + j * 32];
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < NI; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], acc[i][j], 0, 0, 0);
        }

        if (more) store_lds(buf ^ 1);
        __syncthreads();
    }

    // Epilogue: each store instruction writes two 128 B row segments.
#pragma unroll
    for (int i = 0; i < MI; ++i) {
#pragma unroll
        for (int j = 0; j < NI; ++j) {
            const int col = col0 + wave_n * WN + j * 32 + l32;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int row = row0 + wave_m * WM + i * 32 + 8 * (v / 4) + 4 * lhi + (v % 4);
                if (!EDGE || (row < M && col < N)) {
                    float* c = &C[static_cast<size_t>(row) * N + col];
                    *c = epilogue(alpha, acc[i][j][v], beta, c);
                }
            }
        }
    }
}

// ------------------------------------------------- kernel 5, whole tiles --
// The same product for problems made of whole 256 x 256 tiles: global data goes
// straight into LDS (global_load_lds_dwordx4: no staging registers, no LDS
// write instructions), every wave owns a WM x 128 strip of the tile in
// accumulator registers, and one workgroup occupies a CU. The K loop is written
// as phases that run from barrier to barrier with the matrix pipe fed
// throughout.
//
// A vector ALU instruction between two MFMAs delays the second one by about 12
// clocks (measured with one wave per SIMD; LDS reads cost about 5, scalar
// instructions and barriers nothing), so the loop contains none: the direct
// loads take a scalar base and a fixed lane offset (direct_load.h), one load
// behind every fourth MFMA of the first group, pinned there
// with scheduling barriers (bunched loads hold the wave at the memory pipeline).
//
// Wave tile. What is left of those delays (LDS reads, direct loads, the wait at
// the barrier, prologue and write-back of a tile) shows when a SIMD has a single
// wave: 8192^3 ran at 0.952 of the fp32 peak with four waves of 128 x 128 (256
// accumulators each), 0.965 with eight of 64 x 128 and 0.973 with sixteen of
// 32 x 128 (64 accumulators, 124 registers, four waves per SIMD: while one wave
// issues its reads or stores its strip, the others keep the matrix pipe busy);
// 8192 x 8192 x 1024, where the write-back weighs more, 125 -> 134 -> 139.5
// TFLOP/s. The narrow strips read the B operand four times as often from LDS
// (5 reads per 16 MFMAs instead of 8 per 64), which fp32 MFMAs, 64 clocks for
// two registers of operands, leave ample room for. The whole-tile launches use
// 32 x 128.
//
// LDS layout of one K tile (two stages):
//   As[m][k]  as in global memory, BK floats per row. A wave-wide direct load
//             writes 1 KiB of contiguous LDS (lane l lands at base + 16 l), so
//             rows cannot be padded; the 16 B chunk c of row m is kept in slot
//             c ^ ((m >> SWZ) & (chunks - 1)) instead, which spreads the 16 rows
//             a quarter-wave reads with ds_read_b128 over all 64 banks.
//   Bs[k][n]  as in global memory, one 1 KiB row per direct load.
// MFMA operands, per group of 8 k values starting at k8: lane (l32, lhi) reads
// the A chunk k8 + 4 lhi .. + 3 of row l32 (one ds_read_b128 per 32-row block)
// and, for jj = 0..3, B[k8 + 4 lhi + jj][4 l32 .. 4 l32 + 3] (one ds_read_b128
// each). MFMA jj multiplies element jj of the A chunk by element j of the B
// chunk into sub-tile j: the two k values of a 32x32x2 instruction are
// k8 + jj and k8 + 4 + jj, and lane l32 of sub-tile j holds column 4 l32 + j,
// so a lane owns 4 consecutive columns of C and stores them as one 16 B packet.
//
// RAGGED (with EDGE): N and K need not be multiples of 4 and the matrices need only be 4 B aligned. The 16 B
// loads then start at 4 B-aligned addresses, which the memory path accepts, and a descriptor's range check
// is made dword by dword, so that a chunk that straddles an extent's end arrives with its outer dwords
// zeroed (both measured on gfx950). The K loop covers K rounded down to a multiple of 4, where every A
// chunk lies inside its row; a B chunk that straddles the end of a row brings the head of the next row
// into columns >= N, which are never stored. The last K % 4 values of k are added in front of the
// write-back from ordinary loads, and C is written element by element where a chunk straddles N.
//
// STREAMK: the grid is gridDim.x workgroups that share the (tile, K tile) iterations of `sk_tiles` tiles evenly,
// whatever their number: tile number first_big + t for t < sk_tiles, each K_all / BK (rounded up) iterations long,
// laid end to end; workgroup w takes iterations [w I / G, (w + 1) I / G) of the I in all. A workgroup's share is
// a run of segments, each a range of K tiles of one output tile. A segment that covers its tile's whole K range
// is finished here (alpha, beta, C); any other is stored as a raw BM x BN partial product into a slot of the
// workspace `ws` (slot 2 w for the segment a workgroup starts with, 2 w + 1 for the one it ends with), and
// sgemm_stream_k_fixup_kernel adds a tile's partial products in the order of k and finishes the tile. No
// workgroup waits for another one. (The reference's launcher gives every block one whole tile,
// evals/4090_sgemm/runner.cu:191-243; this is the same tile loop entered and left in the middle of K.)
template <int BM, int BN, int BK, int WM, int WN, bool EDGE, bool RAGGED = false, bool STREAMK = false>
__global__ __launch_bounds__((BM / WM) * (BN / WN) * kWave) void sgemm_wave_tile_dma_kernel(
    int M, int N, int K_all, float alpha, const float* __restrict__ A, const float* __restrict__ B,
    float beta, float* C, int tiles_m, int tiles_n, int first_big, float* ws = nullptr, int sk_tiles = 0) {
    static_assert(EDGE || !RAGGED, "the ragged form is an edge form");
    static_assert(!STREAMK || !RAGGED, "the shared-K form needs 16 B-aligned rows");
    // lda: elements between A rows. K: the part of the k range the loops cover.
    const int lda = K_all;
    const int K = RAGGED ? K_all - K_all % 4 : K_all;
    constexpr int WAVES_N = BN / WN;
    constexpr int WAVES = (BM / WM) * WAVES_N;
    constexpr int MI = WM / 32, NI = 4;
    static_assert(WN == 128 && BN == 256, "a lane owns 4 columns of a 128-wide wave tile; a B row is one direct load");
    constexpr int KP = BK / 4;                        // 16 B chunks per A row
    constexpr int SWZ = KP == 4 ? 2 : 1;
    static_assert(KP == 4 || KP == 8, "BK is 16 or 32");
    constexpr int KS = BK / 8;                        // operand groups (8 k values) per tile
    constexpr int ROWS_PER_LOAD = kWave / KP;         // A rows one wave-wide load covers
    constexpr int ROWS_PER_PASS = ROWS_PER_LOAD * WAVES;
    static_assert(BM % ROWS_PER_PASS == 0 && BK % WAVES == 0, "whole load passes");
    constexpr int A_PER = BM / ROWS_PER_PASS, B_PER = BK / WAVES;  // loads per wave per tile
    // MFMAs between two direct loads: the configured gap, or less when the first group is too short for it
    constexpr int WANTED_GAP = 4;
    constexpr int LOAD_GAP = (A_PER + B_PER) * WANTED_GAP <= 4 * MI * 4 ? WANTED_GAP : (4 * MI * 4) / (A_PER + B_PER);
    static_assert(LOAD_GAP >= 1 && (A_PER + B_PER) * LOAD_GAP <= 4 * MI * 4, "the loads of a tile fit among the MFMAs of one group");
    static_assert(((ROWS_PER_PASS >> SWZ) % KP) == 0 && ((32 >> SWZ) % KP) == 0,
                  "the swizzle term must repeat with the load pass and the 32-row MFMA block");

    __shared__ __attribute__((aligned(1024))) float As0[BM * BK];
    __shared__ __attribute__((aligned(1024))) float As1[BM * BK];
    __shared__ __attribute__((aligned(1024))) float Bs0[BK * BN];
    __shared__ __attribute__((aligned(1024))) float Bs1[BK * BN];

    const int tid = threadIdx.x;
    const int lane = tid & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);  // wave-uniform, lives in an SGPR
    const int wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;
    const int l32 = lane & 31, lhi = lane >> 5;

    f32x16 acc[MI][NI];

    // Load side. A: in pass u this wave fills rows [(u * WAVES + wave) * ROWS_PER_LOAD, + ROWS_PER_LOAD);
    // lane l owns row l / KP of those and slot l % KP. The swizzle term is the same in every pass.
    // B: in pass u this wave fills k-row u * WAVES + wave; lane l owns columns 4 l .. 4 l + 3.
    // Addresses are a wave-uniform base (scalar registers, advanced by scalar adds) plus a
    // loop-invariant 32-bit lane offset, so that the K loop holds no vector address arithmetic:
    // a vector ALU instruction between two MFMAs delays the second one.
    const int ld_row = wave * ROWS_PER_LOAD + lane / KP;
    const int ld_chunk = (lane % KP) ^ ((ld_row >> SWZ) & (KP - 1));
    const uint32_t a_lane = (static_cast<uint32_t>(lane / KP) * static_cast<uint32_t>(lda) + ld_chunk * 4) * 4u;  // bytes
    const uint32_t b_lane = static_cast<uint32_t>(lane) * 16u;
    const size_t a_pass = static_cast<size_t>(ROWS_PER_PASS) * lda * 4;
    const size_t b_pass = static_cast<size_t>(WAVES) * N * 4;
    constexpr int LOADS = A_PER + B_PER;

    // Operand side.
    const int sw = (l32 >> SWZ) & (KP - 1);
    int a_off[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) a_off[s] = (wave_m * WM + l32) * BK + ((2 * s + lhi) ^ sw) * 4;
    const int b_off = (4 * lhi) * BN + wave_n * WN + 4 * l32;

    f32x4 fa[2][MI], fb[2][4];
    auto read_frags = [&](const float* as, const float* bs, int s, int slot) {
#pragma unroll
        for (int i = 0; i < MI; ++i) fa[slot][i] = *reinterpret_cast<const f32x4*>(&as[a_off[s] + i * 32 * BK]);
#pragma unroll
        for (int jj = 0; jj < 4; ++jj)
            fb[slot][jj] = *reinterpret_cast<const f32x4*>(&bs[b_off + (8 * s + jj) * BN]);
    };
    // `between(m)` runs after the m-th MFMA of the group.
    auto mfma_all = [&](int slot, auto between) {
#pragma unroll
        for (int jj = 0; jj < 4; ++jj)
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < NI; ++j) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[slot][i][jj], fb[slot][jj][j], acc[i][j], 0, 0, 0);
                    between((jj * MI + i) * NI + j);
                }
    };
    auto nothing = [](int) {};
    using yes = std::integral_constant<bool, true>;
    using no = std::integral_constant<bool, false>;

    // The product of A[row0 .., k_begin .. k_end) and B[k_begin .. k_end, col0 ..) for one BM x BN tile (k_begin a
    // multiple of BK). raw == false: written to C as alpha * product + beta * C. raw == true (STREAMK only): the
    // bare product, stored as a BM x BN array at `part`.
    auto run_tile = [&](const int row0, const int col0, const int k_begin, const int k_end, const bool raw, float* part) {
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int j = 0; j < NI; ++j)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

        const char* a_wave = reinterpret_cast<const char*>(A + static_cast<size_t>(row0 + wave * ROWS_PER_LOAD) * lda);
        const char* b_wave = reinterpret_cast<const char*>(B + static_cast<size_t>(wave) * N + col0);

        // EDGE: M, N, K need not be whole tiles (N and K multiples of 4, so that rows stay 16 B aligned and
        // a 16 B chunk is whole or absent). The loads go through buffer descriptors whose extents end with
        // the matrices: A rows >= M and B rows >= K lie beyond them and arrive as zeros. What lies past
        // the end of a row is the next row, so there the lane offset is replaced by one beyond any extent:
        // B columns >= N (fixed per lane) and, in the partial K tile, A chunks with k >= K.
        const int a_first = row0 + wave * ROWS_PER_LOAD;              // this wave's first A row
        const long long a_left = static_cast<long long>(M - a_first) * lda * 4;
        const long long b_left = (static_cast<long long>(k_end - wave) * N - col0) * 4;
        const i32x4 a_rsrc = buffer_descriptor(EDGE && a_left > 0 ? static_cast<const void*>(a_wave) : static_cast<const void*>(A),
                                               EDGE ? clamped_extent(a_left) : 0u);
        const i32x4 b_rsrc = buffer_descriptor(EDGE && b_left > 0 ? static_cast<const void*>(b_wave) : static_cast<const void*>(B),
                                               EDGE ? clamped_extent(b_left) : 0u);
        const int k_full = k_end - k_end % BK;
        const uint32_t a_tail = (k_full + ld_chunk * 4 < k_end) ? a_lane : kBeyondExtent;
        const uint32_t b_edge = (col0 + 4 * lane < N) ? b_lane : kBeyondExtent;
        // Load number m (0 .. A_PER + B_PER - 1) of the tile that starts at k0.
        auto issue_load = [&](float* as, float* bs, int k0, int m) {
            if constexpr (EDGE) {
                if (m < A_PER)
                    direct_load16_buffer(a_rsrc, k0 < k_full ? a_lane : a_tail,
                                         static_cast<uint32_t>(k0) * 4u + m * static_cast<uint32_t>(a_pass),
                                         as + (m * ROWS_PER_PASS + wave * ROWS_PER_LOAD) * BK);
                else
                    direct_load16_buffer(b_rsrc, b_edge,
                                         (static_cast<uint32_t>(k0) + (m - A_PER) * WAVES) * static_cast<uint32_t>(N) * 4u,
                                         bs + ((m - A_PER) * WAVES + wave) * BN);
            } else {
                if (m < A_PER)
                    direct_load16(a_wave + static_cast<size_t>(k0) * 4 + m * a_pass, a_lane,
                                  as + (m * ROWS_PER_PASS + wave * ROWS_PER_LOAD) * BK);
                else
                    direct_load16(b_wave + static_cast<size_t>(k0) * N * 4 + (m - A_PER) * b_pass, b_lane,
                                  bs + ((m - A_PER) * WAVES + wave) * BN);
            }
        };

        // One phase = everything between two barriers. It is entered right after the
        // barrier that says "tile t is complete in (as, bs), nobody reads (as_n, bs_n)
        // any more", while operand slot 1 still holds the last group of tile t-1:
        //   read group 0 of tile t           -> slot 0
        //   MFMAs of the last group of t-1   <- slot 1, with the direct loads of tile t+1 issued among them
        //   groups 0 .. KS-2 of tile t, each preceded by the reads of the next group
        //   wait for this wave's direct loads, barrier
        auto phase = [&](float* as, float* bs, float* as_n, float* bs_n, int k_next, auto prefetch) {
            read_frags(as, bs, 0, 0);
            mfma_all(1, [&](int m) {
                if constexpr (prefetch) {
                    if (m % LOAD_GAP == 0 && m / LOAD_GAP < LOADS) {
                        issue_load(as_n, bs_n, k_next, m / LOAD_GAP);
                        // The scheduler would otherwise bunch the loads together, and a burst of
                        // them holds the wave (and with it the next MFMA) at the memory pipeline.
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            });
#pragma unroll
            for (int s = 0; s + 1 < KS; ++s) {
                read_frags(as, bs, s + 1, (s + 1) & 1);
                mfma_all(s & 1, nothing);
            }
            constexpr int G = 4 * MI * NI;  // MFMAs per group
            constexpr int PLACED = prefetch ? (LOADS - 1) * LOAD_GAP + 1 : 0;  // MFMAs above the last sched_barrier
            if constexpr (!prefetch) __builtin_amdgcn_sched_group_barrier(0x100, MI + 4, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, G - PLACED, 0);
#pragma unroll
            for (int s = 0; s + 1 < KS; ++s) {
                __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, MI + 4, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, G - 4, 0);
            }
            __builtin_amdgcn_sched_barrier(0);  // keep the MFMAs above the barrier: the direct loads get a whole tile to land
            __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, kLgkmMax));  // the direct loads are invisible to the compiler's wait counts
            __syncthreads();
        };

        // Slot 1 starts as zeros, so the "previous tile" MFMAs of the first phase add nothing.
#pragma unroll
        for (int i = 0; i < MI; ++i) fa[1][i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) fb[1][jj] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

        auto load_tile0 = [&](float* as, float* bs) {
#pragma unroll
            for (int m = 0; m < LOADS; ++m) issue_load(as, bs, k_begin, m);
            __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, kLgkmMax));
            __syncthreads();
        };

        // The launcher guarantees k_end > k_begin and, unless EDGE, whole K tiles. Tiles alternate between the
        // two stages such that the last tile always sits in stage 1.
        const int k_tiles = (k_end - k_begin + BK - 1) / BK;
        int t = 0;
        if (k_tiles & 1) {
            load_tile0(As1, Bs1);
            if (k_tiles > 1) {
                phase(As1, Bs1, As0, Bs0, k_begin + BK, yes{});
                t = 1;
            }
        } else {
            load_tile0(As0, Bs0);
        }
        for (; t + 2 < k_tiles; t += 2) {
            phase(As0, Bs0, As1, Bs1, k_begin + (t + 1) * BK, yes{});
            phase(As1, Bs1, As0, Bs0, k_begin + (t + 2) * BK, yes{});
        }
        if (k_tiles > 1) phase(As0, Bs0, As1, Bs1, k_begin + (t + 1) * BK, yes{});
        phase(As1, Bs1, As0, Bs0, 0, no{});
        mfma_all(1, nothing);  // last group of the last tile

        // Epilogue: a lane holds columns 4 l32 .. 4 l32 + 3 of 16 rows per 32-row block.
        const int c_row = row0 + wave_m * WM + 4 * lhi, c_col = col0 + wave_n * WN + 4 * l32;
        if constexpr (STREAMK) {
            if (raw) {
                // The bare product of this segment, every element of the tile (edge tiles hold zeros outside C).
                float* p_lane = part + static_cast<size_t>(wave_m * WM + 4 * lhi) * BN + wave_n * WN + 4 * l32;
#pragma unroll
                for (int i = 0; i < MI; ++i) {
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int r_in = i * 32 + 8 * (v / 4) + (v % 4);
                        f32x4 r;
#pragma unroll
                        for (int j = 0; j < NI; ++j) r[j] = acc[i][j][v];
                        *reinterpret_cast<f32x4*>(p_lane + static_cast<size_t>(r_in) * BN) = r;
                    }
                }
                return;
            }
        }
        float* c_lane = C + static_cast<size_t>(c_row) * N + c_col;
        auto write_back = [&](auto read_c) {
#pragma unroll
            for (int i = 0; i < MI; ++i) {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int r_in = i * 32 + 8 * (v / 4) + (v % 4);
                    if (EDGE && (c_row + r_in >= M || c_col >= N)) continue;
                    f32x4* c = reinterpret_cast<f32x4*>(c_lane + static_cast<size_t>(r_in) * N);
                    f32x4 r;
                    if constexpr (read_c) {
                        const f32x4 old = *c;
#pragma unroll
                        for (int j = 0; j < NI; ++j) r[j] = __builtin_fmaf(alpha, acc[i][j][v], beta * old[j]);
                    } else {
#pragma unroll
                        for (int j = 0; j < NI; ++j) r[j] = alpha * acc[i][j][v];
                    }
                    *c = r;
                }
                __builtin_amdgcn_sched_barrier(0);  // at most one 32-row block of C reads in flight (64 registers)
            }
        };
        if constexpr (!RAGGED) {
            if (beta == 0.0f) write_back(no{}); else write_back(yes{});
        } else {
            // The k values the loop left out (K_all % 4 of them): a lane adds them to its 16 rows x 4 columns
            // per 32-row block from ordinary loads.
            const int k_tail = K_all - K;
            if (k_tail > 0 && c_col < N) {
                float bt[3][NI];
#pragma unroll
                for (int t = 0; t < 3; ++t)
#pragma unroll
                    for (int j = 0; j < NI; ++j)
                        bt[t][j] = (t < k_tail && c_col + j < N) ? B[static_cast<size_t>(K + t) * N + c_col + j] : 0.0f;
#pragma unroll
                for (int i = 0; i < MI; ++i)
#pragma unroll
                    for (int v = 0; v < 16; ++v) {
                        const int row = c_row + i * 32 + 8 * (v / 4) + (v % 4);
                        if (row >= M) continue;
                        const float* a_row = A + static_cast<size_t>(row) * lda + K;
#pragma unroll
                        for (int t = 0; t < 3; ++t)
                            if (t < k_tail) {
                                const float a = a_row[t];
#pragma unroll
                                for (int j = 0; j < NI; ++j) acc[i][j][v] = __builtin_fmaf(a, bt[t][j], acc[i][j][v]);
                            }
                    }
            }
            // C rows are 4 B aligned only: whole chunks as 16 B accesses at that alignment, the chunk that
            // straddles N element by element.
            typedef float f32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));
            const bool read_c = beta != 0.0f;
#pragma unroll
            for (int i = 0; i < MI; ++i) {
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int r_in = i * 32 + 8 * (v / 4) + (v % 4);
                    if (c_row + r_in >= M || c_col >= N) continue;
                    float* c = c_lane + static_cast<size_t>(r_in) * N;
                    if (c_col + NI <= N) {
                        f32x4_a4* c4 = reinterpret_cast<f32x4_a4*>(c);
                        f32x4 old = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
                        if (read_c) old = *c4;
                        f32x4 r;
#pragma unroll
                        for (int j = 0; j < NI; ++j)
                            r[j] = read_c ? __builtin_fmaf(alpha, acc[i][j][v], beta * old[j]) : alpha * acc[i][j][v];
                        *c4 = r;
                    } else {
#pragma unroll
                        for (int j = 0; j < NI; ++j)
                            if (c_col + j < N)
                                c[j] = read_c ? __builtin_fmaf(alpha, acc[i][j][v], beta * c[j]) : alpha * acc[i][j][v];
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };

    if constexpr (!STREAMK) {
        // first_big < 0: the grid covers the tiles_m x tiles_n grid of BM x BN tiles. Otherwise this launch
        // finishes what a launch on 256 x 256 tiles left over: tiles_m x tiles_n is that launch's grid, first_big
        // the first tile number it did not take, and every leftover tile is cut into 256 / BM row slices.
        int row0, col0;
        if (first_big < 0) {
            int tm, tn;
            xcd_tile_coords(static_cast<int>(blockIdx.x), tiles_m, tiles_n, tm, tn);
            row0 = tm * BM;
            col0 = tn * BN;
        } else {
            constexpr int SUB = 256 / BM;
            int tm, tn;
            xcd_tile_coords(first_big + blockIdx.x / SUB, tiles_m, tiles_n, tm, tn);
            row0 = tm * 256 + static_cast<int>(blockIdx.x % SUB) * BM;
            col0 = tn * 256;
        }
        run_tile(row0, col0, 0, K, false, nullptr);
    } else {
        // This workgroup's run of iterations, segment by segment. Iteration i is K tile i % kt of tile i / kt.
        typedef unsigned long long u64;
        const u64 kt = static_cast<u64>((K + BK - 1) / BK), total = static_cast<u64>(sk_tiles) * kt;
        const u64 w = blockIdx.x, groups = gridDim.x;
        u64 it = w * total / groups;
        const u64 it_end = (w + 1) * total / groups;
        const u64 first_tile = it / kt;
        while (it < it_end) {
            const u64 tile = it / kt, k0 = it - tile * kt;
            const u64 k1 = (it_end - it < kt - k0) ? k0 + (it_end - it) : kt;
            int tm, tn;
            xcd_tile_coords(first_big + static_cast<int>(tile), tiles_m, tiles_n, tm, tn);
            const bool raw = !(k0 == 0 && k1 == kt);
            const int k_end = static_cast<int>(k1 * BK) < K ? static_cast<int>(k1 * BK) : K;
            float* part = ws + (2 * w + (tile != first_tile ? 1u : 0u)) * static_cast<size_t>(BM * BN);
            run_tile(tm * BM, tn * BN, static_cast<int>(k0 * BK), k_end, raw, part);
            it += k1 - k0;
        }
    }
}

// Finishes the tiles whose K range sgemm_wave_tile_dma_kernel<..., STREAMK> shared between workgroups:
// C = alpha * (the tile's partial products, added in the order of k: the same bits on every run) + beta * C. One
// thread per 4 consecutive columns; grid = sk_tiles x (BM * BN / 1024) workgroups of 256. The arithmetic that
// says which workgroup held which part of which tile is the kernel's own.
template <int BM, int BN, int BK>
__global__ __launch_bounds__(256) void sgemm_stream_k_fixup_kernel(int M, int N, int K, float alpha, float beta, float* C,
                                                                   const float* __restrict__ ws, int tiles_m, int tiles_n,
                                                                   int first_tile_number, int sk_tiles, unsigned groups) {
    typedef unsigned long long u64;
    constexpr unsigned PER_TILE = BM * BN / 1024;  // workgroups per tile
    const unsigned tile = blockIdx.x / PER_TILE;
    const unsigned q = (blockIdx.x % PER_TILE) * 256 + threadIdx.x;  // which 16 B packet of the tile
    const int r = static_cast<int>(q / (BN / 4)), c = static_cast<int>(q % (BN / 4)) * 4;
    const u64 kt = static_cast<u64>((K + BK - 1) / BK), total = static_cast<u64>(sk_tiles) * kt;
    const u64 lo = tile * kt, hi = lo + kt;  // the tile's iterations
    // first and last workgroup whose share [w total / groups, (w + 1) total / groups) meets [lo, hi)
    u64 w0 = (lo * groups) / total, w1 = ((hi - 1) * groups) / total;
    while (w0 > 0 && w0 * total / groups > lo) --w0;
    while ((w0 + 1) * total / groups <= lo) ++w0;
    while (w1 + 1 < groups && (w1 + 1) * total / groups < hi) ++w1;
    while (w1 * total / groups >= hi) --w1;
    if (w0 == w1) return;  // one workgroup had the whole K range of this tile and finished it
    int tm, tn;
    xcd_tile_coords(first_tile_number + static_cast<int>(tile), tiles_m, tiles_n, tm, tn);
    const int row = tm * BM + r, col = tn * BN + c;
    if (row >= M || col >= N) return;  // N is a multiple of 4: a packet is inside or outside
    // Four partial products are fetched at a time (the loads are independent of each other), then added in order.
    const float* mine = ws + static_cast<size_t>(r) * BN + c;
    f32x4 sum = {0.0f, 0.0f, 0.0f, 0.0f};
    for (u64 w = w0; w <= w1; w += 4) {
        f32x4 p[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            p[u] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            const u64 begins = (w + u) * total / groups;
            // past the tile's last workgroup, or a workgroup without a share (it wrote nothing): adds +0
            if (w + u > w1 || begins == (w + u + 1) * total / groups) continue;
            const u64 slot = 2 * (w + u) + (begins / kt != tile ? 1u : 0u);
            p[u] = *reinterpret_cast<const f32x4*>(mine + slot * static_cast<size_t>(BM * BN));
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) sum += p[u];
    }
    f32x4* out = reinterpret_cast<f32x4*>(C + static_cast<size_t>(row) * N + col);
    f32x4 res;
    if (beta == 0.0f) {
#pragma unroll
        for (int j = 0; j < 4; ++j) res[j] = alpha * sum[j];
    } else {
        const f32x4 old = *out;
#pragma unroll
        for (int j = 0; j < 4; ++j) res[j] = __builtin_fmaf(alpha, sum[j], beta * old[j]);
    }
    *out = res;
}

// -------------------------------------------- kernel 5, one wave per tile --
// Problems too small to give every CU a 256 x 256 tile: the tile is one wave's
// tile (WT x WT, WT = 64 or 32) and the workgroup is one wave, so there are no
// barriers at all; a CU runs four or more such workgroups side by side. Same
// ingredients as the whole-tile kernel above: direct-to-LDS loads with a scalar
// base, swizzled A rows read 16 B per lane, the k / n permutation that lets a
// lane read NI consecutive B columns per k and own NI consecutive C columns, and
// the previous tile's last MFMA group issued first. The K tiles of 16 travel
// through a ring of STAGES private LDS stages; the loads of tile t + STAGES - 1
// go into the stage of tile t - 1 once this wave's own reads of it have returned
// (lgkmcnt), and a tile is read once this wave's loads of it have (vmcnt).
//
// B stage layout. WT = 64: [k][64], a k-row is 256 B, four rows per direct load.
// WT = 32: a k-row is 128 B, and the two half-waves of an operand read (k and
// k + 4) would hit the same 32 banks; rows k and k + 4 therefore share a 256 B
// line (k & 3 selects the line, bit 2 of k the half), which the load side gets by
// permuting which k-row a lane fetches.
//
// EDGE: M, N, K need not be whole tiles (N and K multiples of 4); edges are zero-filled as in the
// whole-tile kernel above (buffer descriptors that end with the matrices, an out-of-range lane
// offset past a row's end), and the K loop runs over at least STAGES tiles, those beyond K all zeros.
//
// KSPLIT > 1 (whole tiles only): with fewer tiles than SIMDs a tile's K range is cut into KSPLIT equal
// parts, one per wave of a workgroup of KSPLIT waves, each with its own ring; the partial tiles meet in
// LDS and wave 0 adds them in the fixed order 0, 1, ..., KSPLIT - 1 (the same bits on every run) and
// writes C. A K split across workgroups would need a workspace the entry points do not have; this one
// needs none. (128 x 4096 x 4096: 512 tiles of 32 x 32 on 1024 SIMDs, 72 TFLOP/s unsplit.)
//
// RAGGED (with EDGE): rows that are only 4 B aligned (any N and K, matrices at any element), handled as in the
// whole-tile kernel: 16 B loads from 4 B-aligned addresses, a K loop over K rounded down to a multiple of 4, the
// last K % 4 values of k added in front of the write-back, C written element by element.
template <int WT, int STAGES, bool EDGE, int KSPLIT = 1, bool RAGGED = false>
__global__ __launch_bounds__(kWave * KSPLIT) void sgemm_single_wave_kernel(
    int M, int N, int K_all, float alpha, const float* __restrict__ A, const float* __restrict__ B,
    float beta, float* C, int tiles_m, int tiles_n, int first_big, int big_rows = 256) {
    static_assert(EDGE || !RAGGED, "the ragged form is an edge form");
    const int lda = K_all;                                       // elements between A rows
    const int K = RAGGED ? K_all - K_all % 4 : K_all;            // the part of the k range the loop covers
    constexpr int BK = 16, KP = 4, SWZ = 2, KS = 2;
    constexpr int MI = WT / 32, NI = WT / 32;
    static_assert(WT == 32 || WT == 64, "wave tile");
    constexpr int A_LOADS = WT / 16;                  // 16 rows of 64 B per load
    constexpr int B_ROWS_PER_LOAD = 1024 / (WT * 4);  // k-rows per load
    constexpr int B_LOADS = BK / B_ROWS_PER_LOAD;
    constexpr int LOADS = A_LOADS + B_LOADS;
    constexpr int GROUP = 4 * MI * NI;                // MFMAs per group of 8 k values
    static_assert(LOADS <= GROUP, "the loads of a tile fit among the MFMAs of one group");
    static_assert((STAGES - 1) * LOADS < 64, "outstanding loads fit the vmcnt counter");

    static_assert(KSPLIT == 1 || !EDGE, "the K split is written for whole tiles");
    __shared__ __attribute__((aligned(1024))) float As_all[KSPLIT][STAGES][WT * BK];
    __shared__ __attribute__((aligned(1024))) float Bs_all[KSPLIT][STAGES][BK * WT];
    const int wave = KSPLIT == 1 ? 0 : __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) / kWave);
    float (&As)[STAGES][WT * BK] = As_all[wave];
    float (&Bs)[STAGES][BK * WT] = Bs_all[wave];

    // first_big < 0: the grid covers the whole tiles_m x tiles_n grid of WT x WT tiles. Otherwise this
    // launch finishes what a launch of the workgroup kernel on big_rows x 256 tiles (big_rows = 256 or 64)
    // left over: tiles_m x tiles_n is that kernel's grid, first_big the first tile number it did not take,
    // and every leftover tile is cut into (big_rows / WT) x (256 / WT) wave tiles.
    int row0, col0;
    if (first_big < 0) {
        int tm, tn;
        xcd_tile_coords(blockIdx.x, tiles_m, tiles_n, tm, tn);
        row0 = tm * WT;
        col0 = tn * WT;
    } else {
        constexpr int SUB_N = 256 / WT;
        const int per_big = (big_rows / WT) * SUB_N;
        int tm, tn;
        xcd_tile_coords(first_big + static_cast<int>(blockIdx.x) / per_big, tiles_m, tiles_n, tm, tn);
        const int sub = static_cast<int>(blockIdx.x) % per_big;
        row0 = tm * big_rows + (sub / SUB_N) * WT;
        col0 = tn * 256 + (sub % SUB_N) * WT;
    }
    if (EDGE && (row0 >= M || col0 >= N)) return;  // a piece of an edge tile that lies wholly outside C
    const int lane = threadIdx.x % kWave;
    const int l32 = lane & 31, lhi = lane >> 5;
    // This wave's part of K: k_len values starting at k_begin (the launcher makes K / KSPLIT whole K tiles).
    const int k_len = K / KSPLIT, k_begin = wave * k_len;

    f32x16 acc[MI][NI];
#pragma unroll
    for (int i = 0; i < MI; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

    // Load side (lane offsets in bytes, loop-invariant).
    const int a_chunk = (lane % KP) ^ (((lane / KP) >> SWZ) & (KP - 1));
    const uint32_t a_lane = (static_cast<uint32_t>(lane / KP) * static_cast<uint32_t>(lda) + a_chunk * 4) * 4u;
    // B: WT = 64: lane l fetches k-row l / 16, columns 4 (l % 16) ..; WT = 32: LDS position l holds
    // k-row (l / 16) + 4 ((l / 8) & 1), columns 4 (l % 8) .. (see the layout note above).
    const int b_krow = WT == 64 ? lane / 16 : (lane / 16) + 4 * ((lane / 8) & 1);
    const int b_col = WT == 64 ? 4 * (lane % 16) : 4 * (lane % 8);
    const uint32_t b_lane = (static_cast<uint32_t>(b_krow) * static_cast<uint32_t>(N) + b_col) * 4u;
    const char* a_base = reinterpret_cast<const char*>(A + static_cast<size_t>(row0) * lda + k_begin);
    const char* b_base = reinterpret_cast<const char*>(B + static_cast<size_t>(k_begin) * N + col0);
    const i32x4 a_rsrc = buffer_descriptor(a_base, EDGE ? clamped_extent(static_cast<long long>(M - row0) * lda * 4) : 0u);
    const i32x4 b_rsrc = buffer_descriptor(b_base, EDGE ? clamped_extent((static_cast<long long>(K) * N - col0) * 4) : 0u);
    const int k_full = K - K % BK;
    const uint32_t a_tail = (k_full + a_chunk * 4 < K) ? a_lane : kBeyondExtent;
    const uint32_t b_edge = (col0 + b_col < N) ? b_lane : kBeyondExtent;
    auto issue_load = [&](int stage, int k0, int m) {
        if constexpr (EDGE) {
            if (m < A_LOADS)
                direct_load16_buffer(a_rsrc, k0 < k_full ? a_lane : (k0 < K ? a_tail : kBeyondExtent),
                                     (static_cast<uint32_t>(m) * 16u * static_cast<uint32_t>(lda) + k0) * 4u,
                                     &As[stage][m * 16 * BK]);
            else
                direct_load16_buffer(b_rsrc, b_edge,
                                     static_cast<uint32_t>(k0 + (m - A_LOADS) * B_ROWS_PER_LOAD) * static_cast<uint32_t>(N) * 4u,
                                     &Bs[stage][(m - A_LOADS) * B_ROWS_PER_LOAD * WT]);
        } else {
            if (m < A_LOADS)
                direct_load16(a_base + (static_cast<size_t>(m) * 16 * lda + k0) * 4, a_lane, &As[stage][m * 16 * BK]);
            else
                direct_load16(b_base + static_cast<size_t>(k0 + (m - A_LOADS) * B_ROWS_PER_LOAD) * N * 4, b_lane,
                              &Bs[stage][(m - A_LOADS) * B_ROWS_PER_LOAD * WT]);
        }
    };

    // Operand side.
    const int sw = (l32 >> SWZ) & (KP - 1);
    int a_off[KS];
#pragma unroll
    for (int g = 0; g < KS; ++g) a_off[g] = l32 * BK + ((2 * g + lhi) ^ sw) * 4;
    // B element (k = 8 g + 4 lhi + jj, column NI * l32 + j).
    auto b_index = [&](int g, int jj) {
        if constexpr (WT == 64) return (8 * g + 4 * lhi + jj) * WT + NI * l32;
        else return (4 * g + jj) * 64 + lhi * 32 + l32;  // line (k & 3) + 4 (k >> 3), half = bit 2 of k
    };
    typedef float fvec __attribute__((ext_vector_type(NI == 2 ? 2 : 1)));
    f32x4 fa[2][MI];
    float fb[2][4][NI];
    auto read_frags = [&](int stage, int g, int slot) {
#pragma unroll
        for (int i = 0; i < MI; ++i) fa[slot][i] = *reinterpret_cast<const f32x4*>(&As[stage][a_off[g] + i * 32 * BK]);
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
            if constexpr (NI == 2) {
                const fvec b = *reinterpret_cast<const fvec*>(&Bs[stage][b_index(g, jj)]);
                fb[slot][jj][0] = b[0];
                fb[slot][jj][1] = b[1];
            } else {
                fb[slot][jj][0] = Bs[stage][b_index(g, jj)];
            }
        }
    };
    auto mfma_group = [&](int slot, auto after) {
#pragma unroll
        for (int jj = 0; jj < 4; ++jj)
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < NI; ++j) {
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[slot][i][jj], fb[slot][jj][j], acc[i][j], 0, 0, 0);
                    after((jj * MI + i) * NI + j);
                }
    };
    auto nothing = [](int) {};

    // Phase t (tile t sits in stage S): the last group of tile t-1 is multiplied from slot 1 while
    // group 0 of tile t is read into slot 0 and the loads of tile t+STAGES-1 are issued into the
    // stage tile t-1 leaves; then group 0 is multiplied while group 1 is read into slot 1.
    auto phase = [&](auto stage_c, auto prefetch, int k_next) {
        constexpr int S = decltype(stage_c)::value;
        // Reads of tile t-1 have all returned (their values are in slot 1 / were used), so its stage
        // may be overwritten; the explicit wait below keeps that true whatever the compiler schedules.
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(kVmMax, 0));
        __builtin_amdgcn_sched_barrier(0);
        read_frags(S, 0, 0);
        mfma_group(1, [&](int m) {
            if constexpr (prefetch) {
                if (m < LOADS) {
                    issue_load((S + STAGES - 1) % STAGES, k_next, m);
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        });
        read_frags(S, 1, 1);
        mfma_group(0, nothing);
        __builtin_amdgcn_sched_barrier(0);
        // Tile t+1 has landed when at most the loads of the younger tiles are outstanding.
        __builtin_amdgcn_s_waitcnt(waitcnt_imm(prefetch ? (STAGES - 2) * LOADS : 0, kLgkmMax));
        asm volatile("" ::: "memory");  // the compiler does not know that the loads write LDS: no read moves above the wait
        __builtin_amdgcn_sched_barrier(0);
    };
    using yes = std::integral_constant<bool, true>;
    using no = std::integral_constant<bool, false>;

#pragma unroll
    for (int i = 0; i < MI; ++i) fa[1][i] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int jj = 0; jj < 4; ++jj)
#pragma unroll
        for (int j = 0; j < NI; ++j) fb[1][jj][j] = 0.0f;

    // Unless EDGE, the launcher guarantees K % 16 == 0 and at least STAGES tiles. Tile t lives in stage
    // (first + t) % STAGES with `first` chosen such that the last tile sits in the last stage.
    const int k_tiles = EDGE ? ((K + BK - 1) / BK < STAGES ? STAGES : (K + BK - 1) / BK) : k_len / BK;
    const int ragged = k_tiles % STAGES;
    const int first = (STAGES - ragged) % STAGES;
#pragma unroll
    for (int t = 0; t < STAGES - 1; ++t)
#pragma unroll
        for (int m = 0; m < LOADS; ++m) issue_load((first + t) % STAGES, t * BK, m);
    __builtin_amdgcn_s_waitcnt(waitcnt_imm((STAGES - 2) * LOADS, kLgkmMax));
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);

    int k_next = (STAGES - 1) * BK;
    static_assert(STAGES == 4, "the phase sequence below is written out for four stages");
    using s0 = std::integral_constant<int, 0>;
    using s1 = std::integral_constant<int, 1>;
    using s2 = std::integral_constant<int, 2>;
    using s3 = std::integral_constant<int, 3>;
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
    mfma_group(1, nothing);  // last group of the last tile

    if constexpr (KSPLIT > 1) {
        // Partial tiles of waves 1 .. KSPLIT - 1 go through LDS (register v of lane l at [v][l]: no bank
        // conflicts); wave 0 adds them in order and carries on alone.
        __shared__ float partial[KSPLIT - 1][MI * NI * 16][kWave];
        if (wave > 0) {
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < NI; ++j)
#pragma unroll
                    for (int v = 0; v < 16; ++v) partial[wave - 1][(i * NI + j) * 16 + v][lane] = acc[i][j][v];
        }
        __syncthreads();
        if (wave > 0) return;
#pragma unroll
        for (int w = 1; w < KSPLIT; ++w)
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < NI; ++j)
#pragma unroll
                    for (int v = 0; v < 16; ++v) acc[i][j][v] += partial[w - 1][(i * NI + j) * 16 + v][lane];
    }

    // Epilogue: a lane holds columns NI l32 .. NI l32 + NI - 1 of 16 rows per 32-row block.
    float* c_lane = C + static_cast<size_t>(row0 + 4 * lhi) * N + col0 + NI * l32;
    auto write_back = [&](auto read_c) {
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int r_in = i * 32 + 8 * (v / 4) + (v % 4);
                if (EDGE && (row0 + 4 * lhi + r_in >= M || col0 + NI * l32 >= N)) continue;
                float* c = c_lane + static_cast<size_t>(r_in) * N;
                float r[NI];
                if constexpr (read_c) {
                    float old[NI];
                    if constexpr (NI == 2) {
                        const fvec o = *reinterpret_cast<const fvec*>(c);
                        old[0] = o[0];
                        old[1] = o[1];
                    } else {
                        old[0] = *c;
                    }
#pragma unroll
                    for (int j = 0; j < NI; ++j) r[j] = __builtin_fmaf(alpha, acc[i][j][v], beta * old[j]);
                } else {
#pragma unroll
                    for (int j = 0; j < NI; ++j) r[j] = alpha * acc[i][j][v];
                }
                if constexpr (NI == 2) {
                    fvec o;
                    o[0] = r[0];
                    o[1] = r[1];
                    *reinterpret_cast<fvec*>(c) = o;
                } else {
                    *c = r[0];
                }
            }
    };
    if constexpr (!RAGGED) {
        if (beta == 0.0f) write_back(no{}); else write_back(yes{});
    } else {
        const int c_row = row0 + 4 * lhi, c_col = col0 + NI * l32;
        const int k_tail = K_all - K;
        if (k_tail > 0 && c_col < N) {
            float bt[3][NI];
#pragma unroll
            for (int t = 0; t < 3; ++t)
#pragma unroll
                for (int j = 0; j < NI; ++j)
                    bt[t][j] = (t < k_tail && c_col + j < N) ? B[static_cast<size_t>(K + t) * N + c_col + j] : 0.0f;
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int v = 0; v < 16; ++v) {
                    const int row = c_row + i * 32 + 8 * (v / 4) + (v % 4);
                    if (row >= M) continue;
                    const float* a_row = A + static_cast<size_t>(row) * lda + K;
#pragma unroll
                    for (int t = 0; t < 3; ++t)
                        if (t < k_tail) {
                            const float a = a_row[t];
#pragma unroll
                            for (int j = 0; j < NI; ++j) acc[i][j][v] = __builtin_fmaf(a, bt[t][j], acc[i][j][v]);
                        }
                }
        }
        const bool read_c = beta != 0.0f;
#pragma unroll
        for (int i = 0; i < MI; ++i)
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int r_in = i * 32 + 8 * (v / 4) + (v % 4);
                if (c_row + r_in >= M) continue;
                float* c = c_lane + static_cast<size_t>(r_in) * N;
#pragma unroll
                for (int j = 0; j < NI; ++j)
                    if (c_col + j < N)
                        c[j] = read_c ? __builtin_fmaf(alpha, acc[i][j][v], beta * c[j]) : alpha * acc[i][j][v];
            }
    }
}

// ------------------------------------------------ kernel 5, a thin strip of columns --
// C[:, n0 .. n0 + r) = alpha * A @ B[:, n0 .. n0 + r) + beta * C[:, n0 .. n0 + r) for r <= R columns: what is left of
// N beyond a whole number of 256-column tiles when that is a few columns only (N = 4097: a 257th tile column
// would cost a seventeenth of the whole product for one column of C). Not matrix-instruction work: a
// wavefront owns a row of A at a time, its lanes walk the row 64 elements apart (256 B per instruction),
// multiply by the strip of B, which waits in LDS (KC rows of it at a time), and the lanes' sums meet in a
// butterfly. The summation order differs from the big tiles', within the same tolerance.
template <int R, int KC, int ROWS>
__global__ __launch_bounds__(256) void sgemm_thin_columns_kernel(int M, int N, int K, int n0, int r, float alpha,
                                                                 const float* __restrict__ A, const float* __restrict__ B,
                                                                 float beta, float* C) {
    __shared__ float strip[KC * R];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    constexpr int PER_WAVE = ROWS / 4;
    const int row_first = blockIdx.x * ROWS + wave * PER_WAVE;
    float acc[PER_WAVE][R];
#pragma unroll
    for (int i = 0; i < PER_WAVE; ++i)
#pragma unroll
        for (int j = 0; j < R; ++j) acc[i][j] = 0.0f;
    for (int k0 = 0; k0 < K; k0 += KC) {
        const int kc = K - k0 < KC ? K - k0 : KC;
        __syncthreads();  // the strip of the chunk before is no longer read
        // only the r real columns are fetched (the others' sums are never stored); four loads in flight per thread
        for (int e0 = threadIdx.x; e0 < kc * r; e0 += 4 * 256) {
            float b[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int e = e0 + u * 256;
                b[u] = e < kc * r ? B[static_cast<size_t>(k0 + e / r) * N + n0 + e % r] : 0.0f;
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int e = e0 + u * 256;
                if (e < kc * r) strip[(e / r) * R + e % r] = b[u];
            }
        }
        __syncthreads();
        // four steps of 64 k at a time: 4 * PER_WAVE loads in flight per lane
        for (int kb = 0; kb < kc; kb += 4 * kWave) {
            float a[4][PER_WAVE];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int k = kb + u * kWave + lane;
#pragma unroll
                for (int i = 0; i < PER_WAVE; ++i)
                    a[u][i] = (k < kc && row_first + i < M) ? A[static_cast<size_t>(row_first + i) * K + k0 + k] : 0.0f;
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int k = kb + u * kWave + lane;
                if (k < kc) {
#pragma unroll
                    for (int j = 0; j < R; ++j) {
                        const float b = strip[k * R + j];
#pragma unroll
                        for (int i = 0; i < PER_WAVE; ++i) acc[i][j] = __builtin_fmaf(a[u][i], b, acc[i][j]);
                    }
                }
            }
        }
    }
#pragma unroll
    for (int i = 0; i < PER_WAVE; ++i)
#pragma unroll
        for (int j = 0; j < R; ++j) {
            float v = acc[i][j];
#pragma unroll
            for (int d = 32; d >= 1; d >>= 1) v += __shfl_xor(v, d, kWave);
            if (lane == 0 && row_first + i < M && j < r) {
                float* c = &C[static_cast<size_t>(row_first + i) * N + n0 + j];
                *c = epilogue(alpha, v, beta, c);
            }
        }
}

// --------------------------------------------------- kernel 5, a thin strip of rows --
// C[m0 .. m0 + r, :) = alpha * A[m0 .. m0 + r, :) @ B + beta * C[m0 .. m0 + r, :) for r <= R rows: what is left of M
// beyond a whole number of 256-row tiles when that is a few rows only (M = 4097: a 17th tile row would cost a
// seventeenth of the whole product, or a round of its own, for one row of C). A vector-matrix product that reads
// all of B once. A workgroup owns 16 columns (N = 4096 gives every CU one); a wavefront's lanes are four rows of k
// by sixteen columns, so that one load instruction fetches 64 B of four rows of B; its sixteen wavefronts take a
// sixteenth of K each. Lane l fetches A[row][k0 + l] for 64 values of k at a time, and the value a lane needs
// (k0 + 4 u + its row of k) comes to it through the LDS crossbar. The sums meet in a fixed order: the wavefronts'
// in LDS, then the four rows of k. The summation order differs from the big tiles', within the same tolerance.
// (With a lane per column and 64 columns per workgroup the kernel kept a quarter of the CUs busy with one multiply
// and one broadcast per lane, k and row: 56 us for 8 x 4096 x 4096 against 17 this way.)
constexpr int kThinRowsCols = 16;  // columns of C per workgroup of the strip kernel (32: 52 us against 32 for 8 x 4096 x 4096)
template <int R>
__global__ __launch_bounds__(1024) void sgemm_thin_rows_kernel(int N, int K, int m0, int r, float alpha,
                                                               const float* __restrict__ A, const float* __restrict__ B,
                                                               float beta, float* C) {
    constexpr int WAVES = 16, COLS = kThinRowsCols, KQ = kWave / COLS;
    __shared__ float part[WAVES][R][kWave];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = __builtin_amdgcn_readfirstlane(static_cast<int>(threadIdx.x) / kWave);
    const int kq = lane / COLS, c = lane % COLS;
    const int col = blockIdx.x * COLS + c;
    const bool live = col < N;
    const int per = (K + WAVES - 1) / WAVES;
    const int k_begin = wave * per, k_end = (k_begin + per < K) ? k_begin + per : K;
    const float* a_rows = A + static_cast<size_t>(m0) * K;
    const float* b_col = B + (live ? col : 0);
    float acc[R];
#pragma unroll
    for (int i = 0; i < R; ++i) acc[i] = 0.0f;
    for (int k0 = k_begin; k0 < k_end; k0 += kWave) {
        float a[R], b[kWave / KQ];
#pragma unroll
        for (int i = 0; i < R; ++i) a[i] = (i < r && k0 + lane < k_end) ? a_rows[static_cast<size_t>(i) * K + k0 + lane] : 0.0f;
#pragma unroll
        for (int u = 0; u < kWave / KQ; ++u) {
            const int k = k0 + KQ * u + kq;
            b[u] = (live && k < k_end) ? b_col[static_cast<size_t>(k) * N] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < kWave / KQ; ++u)
#pragma unroll
            for (int i = 0; i < R; ++i) acc[i] = __builtin_fmaf(__shfl(a[i], KQ * u + kq, kWave), b[u], acc[i]);
    }
#pragma unroll
    for (int i = 0; i < R; ++i) part[wave][i][lane] = acc[i];
    __syncthreads();
    if (wave < r) {   // wavefront i adds up row i: the wavefronts' shares in the order of k, then the four rows of k
        float v = 0.0f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) v += part[w][wave][lane];
        float sum = v;
#pragma unroll
        for (int q = 1; q < KQ; ++q) sum += __shfl(v, c + q * COLS, kWave);
        if (kq == 0 && live) {
            float* out = &C[static_cast<size_t>(m0 + wave) * N + col];
            *out = epilogue(alpha, sum, beta, out);
        }
    }
}

// --------------------------------------------------------------- launchers --

constexpr int kThinColumns = 8;  // up to this many columns beyond whole 256-column tiles go to the thin-strip kernel
constexpr int kThinRows = 8;     // and up to this many rows beyond whole 256-row tiles to its counterpart

// How many of the last rows of an M x N product kernel 5 leaves to the thin-strip kernel (0: none): a few rows
// beyond a whole number of 256-row tiles, when the rows before still fill three quarters of the CUs with tiles.
int thin_rows_of(int M, int N) {
    const int r = M % 256;
    if (M <= 256 || r == 0 || r > kThinRows || N < 256) return 0;
    return static_cast<long long>(M / 256) * ceil_div(N, 256) * 4 >= 3ll * cu_count() ? r : 0;
}
constexpr int kShortK = 2048;    // up to this K the 256 x 256 tiles of a problem that fills the CUs run as 128 x 256 halves, two to a CU

template <int BM, int BN, int BK, int TM, int TN, bool VEC>
int run_thread_tile(int M, int N, int K, float alpha, const float* A, const float* B, float beta,
                    float* C, hipStream_t s) {
    const int nbm = ceil_div(M, BM), nbn = ceil_div(N, BN);
    const dim3 grid(static_cast<unsigned>(nbm) * nbn), block((BM * BN) / (TM * TN));
    const bool whole = (M % BM == 0) && (N % BN == 0) && (K % BK == 0);
    const bool vec_ok = aligned16(A) && aligned16(B) && aligned16(C) && (K % 4 == 0) && (N % 4 == 0);
    if (whole && (!VEC || vec_ok))
        sgemm_thread_tile_kernel<BM, BN, BK, TM, TN, VEC, false><<<grid, block, 0, s>>>(
            M, N, K, alpha, A, B, beta, C, nbn);
    else
        sgemm_thread_tile_kernel<BM, BN, BK, TM, TN, VEC, true><<<grid, block, 0, s>>>(
            M, N, K, alpha, A, B, beta, C, nbn);
    return check_launch("sgemm_thread_tile_kernel");
}

template <int BM, int BN, int BK, int WM, int WN>
int run_wave_tile(int M, int N, int K, float alpha, const float* A, const float* B, float beta,
                  float* C, hipStream_t s) {
    const int tiles_m = ceil_div(M, BM), tiles_n = ceil_div(N, BN);
    const dim3 grid(static_cast<unsigned>(tiles_m) * tiles_n), block((BM / WM) * (BN / WN) * kWave);
    const bool fast = (M % BM == 0) && (N % BN == 0) && (K % BK == 0) && aligned16(A) && aligned16(B);
    if (fast)
        sgemm_wave_tile_kernel<BM, BN, BK, WM, WN, false><<<grid, block, 0, s>>>(
            M, N, K, alpha, A, B, beta, C, tiles_m, tiles_n);
    else if (static_cast<long long>(BM) * K * 4 >= (1ll << 31) || static_cast<long long>(BK) * N * 4 >= (1ll << 31))
        // The edge path addresses a row panel of A and a K tile of B with 32-bit byte offsets.
        return fail(1, "prism_sgemm: kernel 5 with ragged or unaligned operands needs K < %lld and N < %lld",
                    (1ll << 29) / BM, (1ll << 29) / BK);
    else
        sgemm_wave_tile_kernel<BM, BN, BK, WM, WN, true><<<grid, block, 0, s>>>(
            M, N, K, alpha, A, B, beta, C, tiles_m, tiles_n);
    return check_launch("sgemm_wave_tile_kernel");
}

// Whole-tile kernel when the problem is made of 256 x 256 tiles and there are
// enough of them for three quarters of the CUs. n_cols (a multiple of 256 when given): only the first n_cols
// columns of C are computed; N stays the row length of B and C.
template <int BM, int BN, int BK, int WM, int WN, bool ALLOW_EDGES>
bool try_wave_tile_dma(int M, int N, int K, float alpha, const float* A, const float* B, float beta,
                       float* C, hipStream_t s, int* rc, int n_cols = -1) {
    if (K <= 0) return false;
    if (n_cols < 0) n_cols = N;
    const bool aligned = aligned16(A) && aligned16(B) && aligned16(C);
    const bool whole = aligned && M % BM == 0 && n_cols % BN == 0 && N % 4 == 0 && K % BK == 0;
    // Edges: the kernel's buffer offsets are 32 bits wide (a 256-row panel of A plus one K tile; all of B
    // plus one K tile). Rows that do not stay 16 B aligned (N or K not a multiple of 4, or matrices that
    // are only 4 B aligned) take the ragged form, whose K loop needs at least one group of 4.
    const bool ragged = !whole && (!aligned || N % 4 || K % 4);
    if (!whole && (!ALLOW_EDGES || (ragged && K < 4) ||
                   (static_cast<long long>(BM) + 64) * K * 4 >= (1ll << 31) ||
                   (static_cast<long long>(K) + 64) * N * 4 >= (1ll << 31)))
        return false;
    const int tiles_m = ceil_div(M, BM), tiles_n = ceil_div(n_cols, BN);
    if (static_cast<long long>(tiles_m) * tiles_n * 4 < 3ll * cu_count()) return false;
    if (static_cast<long long>(tiles_m) * tiles_n < cu_count()) {
        // A single, partial round of big tiles costs a full one: four strips per SIMD on the CUs that have a
        // tile. The same output as 64 x 256 tiles is whole rounds of one strip per SIMD (about 8 % dearer per
        // strip: less reuse of operands) plus a partial round that try_half_tile_dma cuts into one-wave tiles.
        // 3584^3: 196 big tiles, or 784 = 3 x 256 + 16 small ones, 3.6 strips against 4 (116 -> 131 TFLOP/s).
        const long long t64 = static_cast<long long>(ceil_div(M, 64)) * tiles_n, cus = cu_count(), left = t64 % cus;
        const double last = left == 0 ? 0.0 : (left * 16 <= 8 * cus && K >= 64) ? ceil_div(left * 16, 4 * cus) * 0.35 : 1.08;
        if ((t64 / cus) * 1.08 + last < 3.7) return false;
    }
    const dim3 block((BM / WM) * (BN / WN) * kWave);
    // Tile counts that do not fill whole rounds of CUs: the 256 x 256 kernel takes the whole rounds, and
    // the tiles of the last, partial round are cut into 64 x 64 wave tiles that spread over all SIMDs
    // (6144^3: 2 rounds + 64 tiles instead of 3 rounds). Not worth it when the last round is nearly full.
    static_assert(BM == 256 && BN == 256, "the leftover launch cuts 256 x 256 tiles");
    const int tiles = tiles_m * tiles_n, cus = cu_count();
    int main_tiles = tiles, leftover_wt = 0;
    const bool lane_offsets_fit = static_cast<long long>(K) * 64 < (1ll << 30) && static_cast<long long>(N) * 64 < (1ll << 30);
    // Short K: a tile's write-back (and the read of C in front of it) is a large part of its time, and with one
    // workgroup per CU nothing runs beside it. As 128 x 256 halves (K tiles of 16, 48 KiB of LDS, eight waves) two
    // workgroups share a CU and drift apart, so that one's write-back overlaps the other's K loop:
    // 4096 x 4096 x 128 95 -> 106 TFLOP/s (81 -> 90 with beta), 8192 x 8192 x 256 126 -> 132 (108 -> 121),
    // 16384 x 16384 x 512 142 -> 144 (130 -> 140); level from K = 4096 up (8192^3 152.3 / 152.2).
    // (The tiles of whole rounds only; a partial last round is cut as for any K, below.)
    const bool short_k = K <= kShortK && tiles >= cus && lane_offsets_fit;
    if (ragged && lane_offsets_fit && tiles > cus && tiles % cus != 0 && K >= 64) {
        // The one-wave kernels have no ragged form: 64 x 256 slices, which cost about 0.27 of a round per
        // slice on the fullest CU (128 x 256 halves cost 0.58 per half, never less), when three to a CU do.
        const int left = tiles % cus;
        if (left * 4 <= 3 * cus) {
            main_tiles = tiles - left;
            leftover_wt = 256;
        }
    }
    if (!ragged && lane_offsets_fit && tiles > cus && tiles % cus != 0 && K >= 64) {
        // Cost of the last round in units of one full round of 256 x 256 tiles: a wave tile of 64 (32)
        // is 1/4 (1/16) of a SIMD's share of a big tile and runs at about 0.87 (0.72) of its rate.
        const int left = tiles % cus, simds = 4 * cus;
        const double cost64 = ceil_div(left * 16, simds) * 0.25 / 0.87;
        const double cost32 = ceil_div(left * 64, simds) * 0.0625 / 0.72;
        if (cost64 < 0.9 || cost32 < 0.9) {
            main_tiles = tiles - left;
            leftover_wt = cost64 <= cost32 ? 64 : 32;
        }
        // Or into 64 x 256 slices of this kernel (K tiles of 16, up to three workgroups to a CU). Measured
        // cost of the last round in full rounds, slices against one-wave tiles: 16 tiles left over 0.27 / 0.15,
        // 33 0.26 / 0.35, 64 0.28 / 0.53, 68 0.51 / 0.35, 132 0.75 / 1.05, 144 0.77 / 0.93, 164 0.76 / 1.06:
        // slices cost about 0.27 per slice on the fullest CU, so they win when they give every CU exactly
        // one, or three where one-wave tiles are no better than a full round.
        const bool one_each = left * 4 <= cus && left * 8 >= cus, three_each = left * 4 > 2 * cus && left * 4 <= 3 * cus;
        if (one_each || three_each) {
            main_tiles = tiles - left;
            leftover_wt = 256;
        }
        // In between, 128 x 256 halves (one workgroup to a CU) cost 0.55-0.6 of a round whatever their number;
        // one-wave tiles cost 0.35 for 68 tiles left over, as much for 73, and 0.9 for 105.
        if (left * 16 >= 5 * cus && left * 2 <= cus) {
            main_tiles = tiles - left;
            leftover_wt = 128;
        }
    }
    // `edge` selects the zero-filling variants of both kernels (sub-tiles that lie wholly outside C exit at once).
    auto launch = [&](auto edge, auto ragged_rows) {
        constexpr bool EDGE = decltype(edge)::value, RAGGED = decltype(ragged_rows)::value;
        if (short_k) {
            sgemm_wave_tile_dma_kernel<128, 256, 16, 32, 128, EDGE, RAGGED><<<dim3(static_cast<unsigned>(main_tiles) * 2), dim3(512), 0, s>>>(
                M, N, K, alpha, A, B, beta, C, tiles_m, tiles_n, 0);
            *rc = check_launch("sgemm_wave_tile_dma_kernel (halves, two to a CU)");
        } else {
            sgemm_wave_tile_dma_kernel<BM, BN, BK, WM, WN, EDGE, RAGGED><<<dim3(static_cast<unsigned>(main_tiles)), block, 0, s>>>(
                M, N, K, alpha, A, B, beta, C, tiles_m, tiles_n, -1);
            *rc = check_launch("sgemm_wave_tile_dma_kernel");
        }
        if (*rc == 0 && leftover_wt == 128) {
            // 128 x 256 halves of the same kernel (one workgroup to a CU for a partial round, two for short K)
            sgemm_wave_tile_dma_kernel<128, 256, 16, 32, 128, EDGE, RAGGED><<<dim3(static_cast<unsigned>(tiles - main_tiles) * 2), dim3(512), 0, s>>>(
                M, N, K, alpha, A, B, beta, C, tiles_m, tiles_n, main_tiles);
            *rc = check_launch("sgemm_wave_tile_dma_kernel (leftover halves)");
        } else if (*rc == 0 && leftover_wt == 256) {
            // 64 x 256 slices of the same kernel, three workgroups to a CU
            sgemm_wave_tile_dma_kernel<64, 256, 16, 32, 128, EDGE, RAGGED><<<dim3(static_cast<unsigned>(tiles - main_tiles) * 4), dim3(256), 0, s>>>(
                M, N, K, alpha, A, B, beta, C, tiles_m, tiles_n, main_tiles);
            *rc = check_launch("sgemm_wave_tile_dma_kernel (leftover slices)");
        } else if constexpr (RAGGED) {
            // no one-wave form for rows that are not 16 B aligned
        } else if (*rc == 0 && leftover_wt == 64) {
            sgemm_single_wave_kernel<64, 4, EDGE><<<dim3(static_cast<unsigned>(tiles - main_tiles) * 16), dim3(kWave), 0, s>>>(
                M, N, K, alpha, A, B, beta, C, tiles_m, tiles_n, main_tiles);
            *rc = check_launch("sgemm_single_wave_kernel");
        } else if (*rc == 0 && leftover_wt == 32) {
            sgemm_single_wave_kernel<32, 4, EDGE><<<dim3(static_cast<unsigned>(tiles - main_tiles) * 64), dim3(kWave), 0, s>>>(
                M, N, K, alpha, A, B, beta, C, tiles_m, tiles_n, main_tiles);
            *rc = check_launch("sgemm_single_wave_kernel");
        }
    };
    if (whole) {
        launch(std::false_type{}, std::false_type{});
    } else if (!ragged) {
        if constexpr (ALLOW_EDGES) launch(std::true_type{}, std::false_type{});
    } else {
        if constexpr (ALLOW_EDGES) launch(std::true_type{}, std::true_type{});
    }
    return true;
}

// Between the one-wave tiles (up to one 64 x 64 tile per SIMD) and the 256 x 256 tiles (from three quarters of
// the CUs up) lies a range in which neither fills the chip: there the same direct-to-LDS kernel runs on
// 128 x 256 tiles (eight waves of 32 x 128, K tiles of 16, 48 KiB of LDS, one workgroup per CU) when those give
// every CU at most one tile, else on 64 x 256 tiles (four waves of 32 x 128, 40 KiB of LDS, 138 registers: three
// workgroups per CU) when those give every CU at most three; in both cases at least half of the CUs get one.
template <int BM, bool ALLOW_EDGES>
bool try_half_tile_dma(int M, int N, int K, float alpha, const float* A, const float* B, float beta,
                       float* C, hipStream_t s, int* rc) {
    constexpr int BN = 256, BK = 16, WM = 32, WN = 128;
    if (K <= 0) return false;
    const bool aligned = aligned16(A) && aligned16(B) && aligned16(C);
    const bool whole = aligned && M % BM == 0 && N % BN == 0 && K % BK == 0;
    const bool ragged = !whole && (!aligned || N % 4 || K % 4);
    if (!whole && (!ALLOW_EDGES || (ragged && K < 4) ||
                   (static_cast<long long>(BM) + 64) * K * 4 >= (1ll << 31) ||
                   (static_cast<long long>(K) + 64) * N * 4 >= (1ll << 31)))
        return false;
    const int tiles_m = ceil_div(M, BM), tiles_n = ceil_div(N, BN);
    const long long tiles = static_cast<long long>(tiles_m) * tiles_n;
    const int cus = cu_count(), simds = 4 * cus;
    // 128 x 256 (two strips per SIMD): when nearly every CU gets a tile. 64 x 256 (one strip per SIMD, three
    // workgroups fit a CU): at most four rounds, at least half of the CUs busy.
    if (BM == 128 ? (tiles > cus || tiles * 8 < 7 * cus) : (tiles > 4 * cus || tiles * 2 < cus)) return false;
    // The unit of work is a wavefront's 32 x 128 strip, and a round of 64 x 256 tiles gives every SIMD one.
    // Tile counts that do not fill whole rounds leave most SIMDs waiting for the few that run one strip more
    // (2304^3: 324 tiles, 0.63 at best), so the tiles of the partial last round are cut into one-wave tiles of
    // 64 or 32 that spread over all SIMDs, as for the 256 x 256 tiles above; a 64 x 64 (32 x 32) wave tile is
    // one strip's (a quarter of one strip's) work at about 0.87 (0.72) of its rate.
    int main_tiles = static_cast<int>(tiles), leftover_wt = 0;
    if (BM == 64 && tiles > cus && tiles % cus != 0 && K >= 64 &&
        static_cast<long long>(K) * 64 < (1ll << 30) && static_cast<long long>(N) * 64 < (1ll << 30)) {
        const int left = static_cast<int>(tiles % cus);
        const double cost64 = ceil_div(left * 4, simds) / 0.87, cost32 = ceil_div(left * 16, simds) * 0.25 / 0.72;
        if (cost64 < 0.9 || cost32 < 0.9) {
            main_tiles = static_cast<int>(tiles) - left;
            leftover_wt = cost64 <= cost32 ? 64 : 32;
        }
    }
    const dim3 grid(static_cast<unsigned>(main_tiles)), block((BM / WM) * (BN / WN) * kWave);
    auto launch = [&](auto edge, auto ragged_rows) {
        constexpr bool EDGE = decltype(edge)::value, RAGGED = decltype(ragged_rows)::value;
        sgemm_wave_tile_dma_kernel<BM, BN, BK, WM, WN, EDGE, RAGGED><<<grid, block, 0, s>>>(M, N, K, alpha, A, B, beta, C, tiles_m, tiles_n, -1);
        *rc = check_launch("sgemm_wave_tile_dma_kernel (128 x 256 or 64 x 256)");
        const unsigned left = static_cast<unsigned>(tiles - main_tiles);
        if (*rc == 0 && leftover_wt == 64) {
            sgemm_single_wave_kernel<64, 4, EDGE, 1, RAGGED><<<dim3(left * 4), dim3(kWave), 0, s>>>(
                M, N, K, alpha, A, B, beta, C, tiles_m, tiles_n, main_tiles, BM);
            *rc = check_launch("sgemm_single_wave_kernel (leftover of 64 x 256 tiles)");
        } else if (*rc == 0 && leftover_wt == 32) {
            sgemm_single_wave_kernel<32, 4, EDGE, 1, RAGGED><<<dim3(left * 16), dim3(kWave), 0, s>>>(
                M, N, K, alpha, A, B, beta, C, tiles_m, tiles_n, main_tiles, BM);
            *rc = check_launch("sgemm_single_wave_kernel (leftover of 64 x 256 tiles)");
        }
    };
    if (whole) {
        launch(std::false_type{}, std::false_type{});
    } else if (!ragged) {
        if constexpr (ALLOW_EDGES) launch(std::true_type{}, std::false_type{});
    } else {
        if constexpr (ALLOW_EDGES) launch(std::true_type{}, std::true_type{});
    }
    return true;
}

// ksplit: waves per tile, each with 1 / ksplit of K (1, 2, or 4 for 32 x 32 tiles); more than 1 only for whole tiles.
template <int WT>
bool try_single_wave(int M, int N, int K, float alpha, const float* A, const float* B, float beta, float* C,
                     hipStream_t s, int* rc, int ksplit = 1) {
    constexpr int STAGES = 4;
    if (K <= 0) return false;
    const bool aligned = aligned16(A) && aligned16(B) && aligned16(C);
    if (static_cast<long long>(K) * 64 >= (1ll << 30) || static_cast<long long>(N) * 64 >= (1ll << 30)) return false;
    const int tiles_m = ceil_div(M, WT), tiles_n = ceil_div(N, WT);
    const dim3 grid(static_cast<unsigned>(tiles_m) * tiles_n);
    if (aligned && M % WT == 0 && N % WT == 0 && K % (16 * ksplit) == 0 && K >= 16 * STAGES * ksplit) {
        if (ksplit == 4 && WT == 32)
            sgemm_single_wave_kernel<32, STAGES, false, 4><<<grid, dim3(4 * kWave), 0, s>>>(
                M, N, K, alpha, A, B, beta, C, tiles_m, tiles_n, -1);
        else if (ksplit == 2)
            sgemm_single_wave_kernel<WT, STAGES, false, 2><<<grid, dim3(2 * kWave), 0, s>>>(
                M, N, K, alpha, A, B, beta, C, tiles_m, tiles_n, -1);
        else if (ksplit == 1)
            sgemm_single_wave_kernel<WT, STAGES, false><<<grid, dim3(kWave), 0, s>>>(
                M, N, K, alpha, A, B, beta, C, tiles_m, tiles_n, -1);
        else
            return false;
        *rc = check_launch("sgemm_single_wave_kernel");
        return true;
    }
    if (ksplit != 1) return false;
    // Ragged edges: all of B plus the padding K tiles is addressed with 32-bit byte offsets. Rows that do not
    // stay 16 B aligned take the ragged form, whose K loop needs at least one group of 4.
    if ((static_cast<long long>(K) + 16 * STAGES) * N * 4 >= (1ll << 31)) return false;
    if (!aligned || N % 4 || K % 4) {
        if (K < 4) return false;
        sgemm_single_wave_kernel<WT, STAGES, true, 1, true><<<grid, dim3(kWave), 0, s>>>(
            M, N, K, alpha, A, B, beta, C, tiles_m, tiles_n, -1);
        *rc = check_launch("sgemm_single_wave_kernel (ragged rows)");
        return true;
    }
    sgemm_single_wave_kernel<WT, STAGES, true><<<grid, dim3(kWave), 0, s>>>(
        M, N, K, alpha, A, B, beta, C, tiles_m, tiles_n, -1);
    *rc = check_launch("sgemm_single_wave_kernel (edges)");
    return true;
}

// What prism_sgemm_ws does with a workspace: the K ranges of some or all output tiles are shared evenly between
// `groups` workgroups (the STREAMK form of the workgroup kernel), which takes 2 * groups tile-sized slots of
// workspace for the partial products.
//   bm == 256: problems of 256 x 256 tiles whose count is not a whole number of rounds of the CUs. The whole
//              rounds (main_tiles tiles) run as ever, one tile per workgroup; the sk_tiles tiles of the last,
//              partial round are shared between all CUs, so that round costs its share of a round instead of a
//              whole one (or of what the cheaper cuts of launch_sgemm make of it).
//   bm == 64:  skinny problems (few 64 x 256 tiles, long K; 128 x 4096 x 4096 has 32 such tiles for 256 CUs).
struct StreamKPlan {
    int bm = 0;          // 0: no sharing, the call is launch_sgemm
    int main_tiles = 0;  // tiles of the whole rounds (bm == 256)
    int sk_tiles = 0;
    int groups = 0;
    bool whole = false;  // whole tiles and whole K tiles: the kernel's form without range checks
    size_t bytes() const { return static_cast<size_t>(2) * groups * bm * 256 * sizeof(float); }
};

// The skinny case: a small model of the shared and the unshared kernels says whether sharing pays. Returns the
// number of K parts per tile the model prefers (0: leave it). M, N multiples of 64 and 256, K of 16.
int skinny_parts(int M, int N, int K) {
    if (M <= 0 || N <= 0 || K < 1024 || M % 64 || N % 256 || K % 16) return 0;
    const long long tiles = static_cast<long long>(M / 64) * (N / 256);
    const int cus = cu_count();
    if (tiles * 5 > cus) return 0;                       // from about a fifth of the CUs up the unshared kernels are level
    if (static_cast<long long>(K) * 64 >= (1ll << 30) || static_cast<long long>(N) * 64 >= (1ll << 30)) return 0;
    // Rounds of workgroups, each as long as its part of K plus a fixed cost worth about 128 k (53 ns per k for a
    // wavefront's strip at the fp32 MFMA rate), and the adding-up, which moves parts + 2 times the output at
    // about 5 TB/s behind a second launch. Measured against it on 128 x 4096 x 4096: 4 / 8 / 16 parts
    // 65 / 100 / 93 TFLOP/s (model 65 / 105 / 84).
    int parts = 0;
    double best = 0.0;
    for (int p = 2; p <= 64; p *= 2) {
        if (K % (16 * p) != 0 || K / p < 128) break;
        const double rounds = static_cast<double>(tiles * p) / cus;
        const double us = (rounds < 1.0 ? 1.0 : rounds) * (K / p + 128) * 0.053 + (p + 2) * (static_cast<double>(M) * N * 4.0) / 5.0e6 + 3.0;
        if (parts == 0 || us < best) {
            best = us;
            parts = p;
        }
    }
    // Against the unshared one-wave tiles of 32 x 32, which such shapes take: bound by their L2 traffic (1 B per
    // 8 flop at about 9 TB/s) or by the instructions a wavefront issues one after the other (13.3 ns per k and
    // tile, K cut four or two ways inside the workgroup where launch_sgemm does that), plus about 6 us.
    // Measured: 128 x 4096 x 4096 68 us (model 60), 64 x 512 x 2048 12 (13), 64 x 256 x 16384 65 (60).
    const double flop = 2.0 * M * N * static_cast<double>(K);
    const long long tiles32 = static_cast<long long>(M / 32) * (N / 32), simds = 4ll * cus;
    const int inner = (tiles32 * 8 <= simds && K >= 1024) ? 4 : (tiles32 * 4 <= simds && K >= 512) ? 2 : 1;
    const double chain_us = static_cast<double>((tiles32 * inner + simds - 1) / simds) * (K / inner) * 0.0133;
    const double unshared_us = std::max(flop / 8.0 / 9.0e6, chain_us) + 6.0;
    return (parts >= 2 && best < 0.85 * unshared_us) ? parts : 0;
}

// aligned: A, B and C are 16 B aligned (a query without pointers assumes so).
StreamKPlan stream_k_plan(int M, int N, int K, bool aligned) {
    StreamKPlan plan;
    if (M <= 0 || N <= 0 || K <= 0 || !aligned || N % 4 || K % 4) return plan;  // rows must stay 16 B aligned
    M -= thin_rows_of(M, N);   // the plan is for the rows the tiles keep (launch_sgemm_ws hands the rest to the strip kernel)
    const int cus = cu_count();
    if (const int parts = skinny_parts(M, N, K)) {
        const long long tiles = static_cast<long long>(M / 64) * (N / 256);
        plan.bm = 64;
        plan.sk_tiles = static_cast<int>(tiles);
        plan.groups = static_cast<int>(std::min<long long>(cus, tiles * parts));
        plan.whole = true;
        return plan;
    }
    // 256 x 256 tiles: the same limits as try_wave_tile_dma (32-bit buffer offsets in the range-checked form).
    const bool whole = M % 256 == 0 && N % 256 == 0 && K % 32 == 0;
    if (!whole && ((256ll + 64) * K * 4 >= (1ll << 31) || (static_cast<long long>(K) + 64) * N * 4 >= (1ll << 31))) return plan;
    const long long tiles = static_cast<long long>(ceil_div(M, 256)) * ceil_div(N, 256);
    // Fewer tiles than CUs: sharing all of them was measured level with or behind the smaller tiles launch_sgemm
    // picks there (3072^3 134 against 149 TFLOP/s, 3584^3 139 against 142, 3200^3 125 against 123): every tile
    // then pays for partial products.
    // A short K leaves too little work per tile to pay for partial products and the second launch (5120 x 5120 x K,
    // plain / shared: K = 512 124 / 111, 1024 131 / 128 (4352^2), 2048 134 / 140, 5120 136 / 148 TFLOP/s).
    if (tiles <= cus || tiles > 0x3fffffff || K < kShortK) return plan;
    const int left = static_cast<int>(tiles % cus);
    if (left == 0) return plan;
    // A last round that is nearly full gains nothing from being shared (the partial products cost a few per
    // cent), and one of just under a quarter of the CUs is as cheap as 64 x 256 slices, one to a CU, which
    // launch_sgemm makes of it (6144^3, 64 tiles left: 152.7 against 151.4 shared; 4352^3, 33 left: 136.6
    // against 146.7 shared).
    if (left * 16 > 15 * cus || (left * 4 <= cus && left * 16 >= 3 * cus)) return plan;
    plan.bm = 256;
    plan.main_tiles = static_cast<int>(tiles - left);
    plan.sk_tiles = left;
    plan.groups = cus;
    plan.whole = whole;
    return plan;
}

}  // namespace

size_t sgemm_workspace_bytes(int M, int N, int K) { return stream_k_plan(M, N, K, true).bytes(); }

int sgemm_ws_plan(int M, int N, int K, size_t ws_bytes, int* groups, int* sk_tiles) {
    const StreamKPlan plan = stream_k_plan(M, N, K, true);
    const bool taken = plan.bm != 0 && ws_bytes >= plan.bytes();
    if (groups) *groups = taken ? plan.groups : 0;
    if (sk_tiles) *sk_tiles = taken ? plan.sk_tiles : 0;
    return 0;
}

int launch_sgemm_ws(int variant, int M, int N, int K, float alpha, const float* A, const float* B, float beta,
                    float* C, void* ws, size_t ws_bytes, hipStream_t s) {
    if (int rc = check_sgemm_arguments(variant, M, N, K, A, B, C)) return rc;
    if ((variant == 0 || variant == 5) && M > 0 && N > 0 && K > 0 && ws != nullptr && aligned16(ws)) {
        const StreamKPlan plan = stream_k_plan(M, N, K, aligned16(A) && aligned16(B) && aligned16(C));
        if (const int r = thin_rows_of(M, N); r != 0 && plan.bm != 0 && ws_bytes >= plan.bytes()) {
            if (int rc = launch_sgemm_ws(variant, M - r, N, K, alpha, A, B, beta, C, ws, ws_bytes, s)) return rc;
            sgemm_thin_rows_kernel<kThinRows><<<dim3(static_cast<unsigned>(ceil_div(N, kThinRowsCols))), dim3(1024), 0, s>>>(
                N, K, M - r, r, alpha, A, B, beta, C);
            return check_launch("sgemm_thin_rows_kernel");
        }
        if (plan.bm != 0 && ws_bytes >= plan.bytes()) {
            float* parts = static_cast<float*>(ws);
            const dim3 grid(static_cast<unsigned>(plan.groups));
            if (plan.bm == 64) {
                const int tiles_m = M / 64, tiles_n = N / 256;
                // K tiles of 32 when K allows: a workgroup streams its whole share of B once, and what it has in
                // flight (one stage) is what hides the memory latency; 20 KiB (K tiles of 16) do not.
                if (K % 32 == 0) {
                    sgemm_wave_tile_dma_kernel<64, 256, 32, 32, 128, false, false, true><<<grid, dim3(256), 0, s>>>(
                        M, N, K, alpha, A, B, beta, C, tiles_m, tiles_n, 0, parts, plan.sk_tiles);
                    if (int rc = check_launch("sgemm_wave_tile_dma_kernel (K shared, 64 x 256 tiles)")) return rc;
                    sgemm_stream_k_fixup_kernel<64, 256, 32><<<dim3(static_cast<unsigned>(plan.sk_tiles) * 16), dim3(256), 0, s>>>(
                        M, N, K, alpha, beta, C, parts, tiles_m, tiles_n, 0, plan.sk_tiles, grid.x);
                    return check_launch("sgemm_stream_k_fixup_kernel");
                }
                sgemm_wave_tile_dma_kernel<64, 256, 16, 32, 128, false, false, true><<<grid, dim3(256), 0, s>>>(
                    M, N, K, alpha, A, B, beta, C, tiles_m, tiles_n, 0, parts, plan.sk_tiles);
                if (int rc = check_launch("sgemm_wave_tile_dma_kernel (K shared, 64 x 256 tiles)")) return rc;
                sgemm_stream_k_fixup_kernel<64, 256, 16><<<dim3(static_cast<unsigned>(plan.sk_tiles) * 16), dim3(256), 0, s>>>(
                    M, N, K, alpha, beta, C, parts, tiles_m, tiles_n, 0, plan.sk_tiles, grid.x);
                return check_launch("sgemm_stream_k_fixup_kernel");
            }
            const int tiles_m = ceil_div(M, 256), tiles_n = ceil_div(N, 256);
            if (plan.main_tiles > 0) {
                const dim3 main_grid(static_cast<unsigned>(plan.main_tiles));
                const dim3 halves_grid(static_cast<unsigned>(plan.main_tiles) * 2);  // short K: see try_wave_tile_dma
                if (K <= kShortK && plan.whole)
                    sgemm_wave_tile_dma_kernel<128, 256, 16, 32, 128, false><<<halves_grid, dim3(512), 0, s>>>(
                        M, N, K, alpha, A, B, beta, C, tiles_m, tiles_n, 0);
                else if (K <= kShortK)
                    sgemm_wave_tile_dma_kernel<128, 256, 16, 32, 128, true><<<halves_grid, dim3(512), 0, s>>>(
                        M, N, K, alpha, A, B, beta, C, tiles_m, tiles_n, 0);
                else if (plan.whole)
                    sgemm_wave_tile_dma_kernel<256, 256, 32, 32, 128, false><<<main_grid, dim3(1024), 0, s>>>(
                        M, N, K, alpha, A, B, beta, C, tiles_m, tiles_n, -1);
                else
                    sgemm_wave_tile_dma_kernel<256, 256, 32, 32, 128, true><<<main_grid, dim3(1024), 0, s>>>(
                        M, N, K, alpha, A, B, beta, C, tiles_m, tiles_n, -1);
                if (int rc = check_launch("sgemm_wave_tile_dma_kernel (whole rounds)")) return rc;
            }
            if (plan.whole)
                sgemm_wave_tile_dma_kernel<256, 256, 32, 32, 128, false, false, true><<<grid, dim3(1024), 0, s>>>(
                    M, N, K, alpha, A, B, beta, C, tiles_m, tiles_n, plan.main_tiles, parts, plan.sk_tiles);
            else
                sgemm_wave_tile_dma_kernel<256, 256, 32, 32, 128, true, false, true><<<grid, dim3(1024), 0, s>>>(
                    M, N, K, alpha, A, B, beta, C, tiles_m, tiles_n, plan.main_tiles, parts, plan.sk_tiles);
            if (int rc = check_launch("sgemm_wave_tile_dma_kernel (K shared, 256 x 256 tiles)")) return rc;
            sgemm_stream_k_fixup_kernel<256, 256, 32><<<dim3(static_cast<unsigned>(plan.sk_tiles) * 64), dim3(256), 0, s>>>(
                M, N, K, alpha, beta, C, parts, tiles_m, tiles_n, plan.main_tiles, plan.sk_tiles, grid.x);
            return check_launch("sgemm_stream_k_fixup_kernel");
        }
    }
    return launch_sgemm(variant, M, N, K, alpha, A, B, beta, C, s);
}

int check_sgemm_arguments(int variant, int M, int N, int K, const float* A, const float* B, const float* C) {
    if (variant < 0 || variant > 6) return fail(1, "prism_sgemm: unknown kernel number %d", variant);
    if (M < 0 || N < 0 || K < 0) return fail(1, "prism_sgemm: negative dimension (%d,%d,%d)", M, N, K);
    if (M == 0 || N == 0) return 0;
    if (C == nullptr || (K > 0 && (A == nullptr || B == nullptr)))
        return fail(1, "prism_sgemm: null matrix pointer");
    if (!aligned4(A) || !aligned4(B) || !aligned4(C))
        return fail(1, "prism_sgemm: matrices must be 4-byte aligned");
    return 0;
}

int launch_sgemm(int variant, int M, int N, int K, float alpha, const float* A, const float* B,
                 float beta, float* C, hipStream_t s) {
    if (int rc = check_sgemm_arguments(variant, M, N, K, A, B, C)) return rc;
    if (M == 0 || N == 0) return 0;
    const size_t mn = static_cast<size_t>(M) * N;
    if (variant == 0) variant = 5;
    // K == 0 leaves C = beta * C; the naive kernel does exactly that.
    if (K == 0) variant = 1;

    switch (variant) {
        case 1: {
            const size_t blocks = ceil_div(mn, size_t{256});
            if (blocks > 0x7fffffffull) return fail(1, "prism_sgemm: M*N too large for kernel 1");
            sgemm_naive_kernel<<<dim3(static_cast<unsigned>(blocks)), dim3(256), 0, s>>>(M, N, K, alpha, A, B, beta, C);
            return check_launch("sgemm_naive_kernel");
        }
        case 2: {
            const size_t blocks = static_cast<size_t>(ceil_div(M, 32)) * ceil_div(N, 32);
            sgemm_coalesced_kernel<<<dim3(static_cast<unsigned>(blocks)), dim3(1024), 0, s>>>(M, N, K, alpha, A, B, beta, C);
            return check_launch("sgemm_coalesced_kernel");
        }
        case 3: {
            const int nbn = ceil_div(N, 32);
            const size_t blocks = static_cast<size_t>(ceil_div(M, 32)) * nbn;
            sgemm_lds_block_kernel<<<dim3(static_cast<unsigned>(blocks)), dim3(1024), 0, s>>>(M, N, K, alpha, A, B, beta, C, nbn);
            return check_launch("sgemm_lds_block_kernel");
        }
        case 4:
            // Tile choice of run_my_sgemm_4 (evals/4090_sgemm/runner.cu:163-189).
            if (M >= 128 && N >= 128) return run_thread_tile<128, 128, 8, 8, 8, true>(M, N, K, alpha, A, B, beta, C, s);
            return run_thread_tile<64, 64, 8, 8, 8, true>(M, N, K, alpha, A, B, beta, C, s);
        case 6:
            if (M >= 128 && N >= 128) return run_thread_tile<128, 128, 8, 8, 8, false>(M, N, K, alpha, A, B, beta, C, s);
            return run_thread_tile<64, 64, 8, 8, 8, false>(M, N, K, alpha, A, B, beta, C, s);
        case 5:
            // BM = BN = 128, BK = 16, WM = WN = 64: the tile shape of
            // run_my_sgemm_5 (evals/4090_sgemm/runner.cu:194-202), with four
            // 64-lane waves in place of four 32-lane warps.
            {
                // A few rows beyond a whole number of 256-row tiles (M = 4097) would cost a whole tile row: the
                // product of the rows before runs as ever (the same call on M - r rows), a thin-strip kernel
                // takes the rest (4097 x 4097 x 1025: 108 -> 131 TFLOP/s).
                if (const int r = thin_rows_of(M, N)) {
                    if (int rc = launch_sgemm(5, M - r, N, K, alpha, A, B, beta, C, s)) return rc;
                    sgemm_thin_rows_kernel<kThinRows><<<dim3(static_cast<unsigned>(ceil_div(N, kThinRowsCols))), dim3(1024), 0, s>>>(
                        N, K, M - r, r, alpha, A, B, beta, C);
                    return check_launch("sgemm_thin_rows_kernel");
                }
                // Whole 256 x 256 tiles for at least three quarters of the CUs: the direct-to-LDS kernel,
                // K tiles of 32 (128 KiB of LDS) when K allows, else of 16.
                int rc = 0;
                // A few columns beyond a whole number of 256-column tiles (N = 4097) would cost a whole tile
                // column: the big tiles take the whole columns, a thin-strip kernel the rest.
                if (const int r = N % 256; N > 256 && r > 0 && r <= kThinColumns && M >= 64 &&
                    try_wave_tile_dma<256, 256, 32, 32, 128, true>(M, N, K, alpha, A, B, beta, C, s, &rc, N - r)) {
                    if (rc != 0) return rc;
                    constexpr int ROWS = 8;  // two rows per wavefront: a thousand workgroups for M = 8191
                    sgemm_thin_columns_kernel<kThinColumns, 1024, ROWS><<<dim3(static_cast<unsigned>(ceil_div(M, ROWS))), dim3(256), 0, s>>>(
                        M, N, K, N - r, r, alpha, A, B, beta, C);
                    return check_launch("sgemm_thin_columns_kernel");
                }
                // Ragged M, N, K take the K-tile-of-32 kernel with zero-filled edges (its ragged form when
                // rows are not 16 B aligned).
                if (try_wave_tile_dma<256, 256, 32, 32, 128, true>(M, N, K, alpha, A, B, beta, C, s, &rc)) return rc;
                if (try_wave_tile_dma<256, 256, 16, 32, 128, false>(M, N, K, alpha, A, B, beta, C, s, &rc)) return rc;
                // Small problems (at most one 64 x 64 tile per SIMD): one wave per tile, 32 x 32 tiles when
                // 64 x 64 ones would leave SIMDs without work. In between, the direct-to-LDS kernel on
                // 128 x 256 tiles (at most one per CU) or 64 x 256 tiles (at most three per CU); what is left
                // (K < 4, offsets that do not fit 32 bits) goes to the general kernel.
                const long long simds = 4ll * cu_count();
                const long long tiles64 = static_cast<long long>(ceil_div(M, 64)) * ceil_div(N, 64);
                // A single round of 64 x 256 workgroup tiles that fills at least three quarters of the CUs (one
                // strip per SIMD, operands shared through LDS) is ahead of one-wave tiles over the same output:
                // 2048^3 119 -> 132, 1920 x 2048 x 2048 100 -> 133, 1664 x 2048 x 1024 86 -> 109 TFLOP/s on one box;
                // with fewer tiles it is not (1536^3, 144 tiles: 100 -> 79).
                {
                    const long long t64x256 = static_cast<long long>(ceil_div(M, 64)) * ceil_div(N, 256);
                    if (t64x256 <= cu_count() && t64x256 * 4 >= 3ll * cu_count() &&
                        try_half_tile_dma<64, true>(M, N, K, alpha, A, B, beta, C, s, &rc)) return rc;
                }
                if (tiles64 <= simds) {
                    // Far fewer 32 x 32 tiles than SIMDs: cut K inside the workgroup (2 or 4 waves per tile) as
                    // long as every wave keeps at least 256 of K and at most half of the SIMDs end up with a
                    // wave: 32 x 32 wave tiles move 1 B from L2 per 8 flop, and with a wave on every SIMD that
                    // traffic, not the matrix pipe, is the limit (128 x 4096 x 4096: 72 TFLOP/s with 512 waves,
                    // 65 with 1024). 512^3: 24 -> 35 TFLOP/s, 256 x 256 x 4096: 29 (rocBLAS 13 and 23).
                    const long long tiles32 = static_cast<long long>(ceil_div(M, 32)) * ceil_div(N, 32);
                    if (tiles32 * 8 <= simds && K >= 4 * 256 && try_single_wave<32>(M, N, K, alpha, A, B, beta, C, s, &rc, 4)) return rc;
                    if (tiles32 * 4 <= simds && K >= 2 * 256 && try_single_wave<32>(M, N, K, alpha, A, B, beta, C, s, &rc, 2)) return rc;
                    if (tiles64 < simds && try_single_wave<32>(M, N, K, alpha, A, B, beta, C, s, &rc)) return rc;
                    if (try_single_wave<64>(M, N, K, alpha, A, B, beta, C, s, &rc)) return rc;
                }
                if (try_half_tile_dma<128, true>(M, N, K, alpha, A, B, beta, C, s, &rc)) return rc;
                if (try_half_tile_dma<64, true>(M, N, K, alpha, A, B, beta, C, s, &rc)) return rc;
            }
            return run_wave_tile<128, 128, 16, 64, 64>(M, N, K, alpha, A, B, beta, C, s);  // BM, BN, BK, WM, WN
    }
    return fail(1, "prism_sgemm: unknown kernel number %d", variant);
}

}  // namespace prism
