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
#include "common.h"
#include "tile_map.h"

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

    const int k_tiles = (K + BK - 1) / BK;
    load_global(0);
    store_lds(0);
    __syncthreads();

    for (int t = 0; t < k_tiles; ++t) {
        const int buf = t & 1;
        const bool more = (t + 1 < k_tiles);
        if (more) load_global((t + 1) * BK);

        const uint16_t* ps = &Ps[buf * P_TILE + (wave_m * WM + l32) * LD + lhi * 8];
        const uint16_t* qs = &Qs[buf * Q_TILE + (wave_n * WN + l32) * LD + lhi * 8];
#pragma unroll
        for (int kk = 0; kk < BK; kk += 16) {
            bf16x8 a[MI], b[NI];
#pragma unroll
            for (int i = 0; i < MI; ++i)
                a[i] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(&ps[i * 32 * LD + kk]));
#pragma unroll
            for (int j = 0; j < NI; ++j)
                b[j] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(&qs[j * 32 * LD + kk]));
#pragma unroll
            for (int i = 0; i < MI; ++i)
#pragma unroll
                for (int j = 0; j < NI; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
        }

        if (more) store_lds(buf ^ 1);
        __syncthreads();
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
    if (fast) return launch(gemm_bf16_kernel<BM, BN, BK, WM, WN, false, OutT>);
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
    if (D_f32) return run_gemm_bf16<128, 128, 64, 64, 64, float>(M, N, K, A, B, D_f32, s);
    // Column-major M x N == row-major N x M of B @ A^T.
    return run_gemm_bf16<128, 128, 64, 64, 64, uint16_t>(N, M, K, B, A, C_bf16_colmajor, s);
}

}  // namespace prism
