/*
 * prism_oracle.c - CPU restatement of the reference's algorithms for the
 * add_m / scan / sgemm / bf16-gemm path.
 *
 * TEST INFRASTRUCTURE ONLY. Nothing in the product (prism_amd/, the shared
 * library, include/) may call, link or import this file. It exists so that
 * tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg can check
 * and time-compare the HIP kernels. Plain C99, single-threaded, no GPU.
 *
 * Every function cites the reference file:line it follows
 * (paths inside manya-bansal/prism).
 *
 * How each function is pinned (see tests/test_oracle.py):
 *   oracle_add_m            closed form y = x + m on hand-computed wrap cases; numpy int32 add
 *   oracle_scan_cpu         closed forms (all-ones -> i+1, wrap cases), numpy.cumsum(int32),
 *                           difference invariant out[i]-out[i-1] == x[i]
 *   oracle_scan_exclusive_cpu  closed forms (all-ones -> i, wrap), inclusive[i] - x[i], shifted numpy.cumsum
 *   oracle_scan_max_cpu     closed forms (rising -> itself, falling -> first element, INT32_MIN / INT32_MAX),
 *                           numpy.maximum.accumulate, monotone and out[i] >= x[i] with equality where out steps
 *   oracle_segmented_scan_cpu  no heads -> oracle_scan_cpu; every element a head -> the input; hand-computed
 *                           case with wrap; per-segment numpy.cumsum; the closed form through one global cumsum
 *   oracle_scan_i64_cpu     closed forms (all-ones -> i+1, wrap at 2^63), numpy.cumsum(int64)
 *   oracle_scan_lookback    equality with oracle_scan_cpu on the reference's own test sizes
 *                           and distribution; tail beyond the last full block left untouched
 *   oracle_sgemm_fma        brute-force exact rational/fp64 check on small integer-valued
 *                           inputs where every fma is exact; identity/alpha/beta special cases
 *   oracle_sgemm_f64        numpy float64 matmul; same special cases
 *   oracle_f32_to_bf16      hand-computed tie/NaN/Inf vectors; torch.bfloat16 conversion
 *   oracle_gemm_bf16_f64    numpy float64 matmul of the widened inputs
 * The reference tree holds no numeric golden vectors for this path (its GEMM
 * checks compare against cuBLAS at run time), so none are used.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------ add_m */

/* y[tid] = x[tid] + m, int32 (README.md:133-140, examples/add_m_thread.py:10-19).
 * Wrap-around is made explicit through unsigned arithmetic. */
void oracle_add_m(const int32_t* x, int32_t* y, int32_t m, size_t n) {
    for (size_t i = 0; i < n; ++i) y[i] = (int32_t)((uint32_t)x[i] + (uint32_t)m);
}

/* ------------------------------------------------------------------- scan */

/* The reference's own CPU oracle, verbatim in meaning
 * (evals/4090_scan/scan_harness.cuh:30-36): serial uint32 accumulator. */
void oracle_scan_cpu(size_t n, const uint32_t* x, uint32_t* out) {
    uint32_t accumulator = 0;
    for (size_t i = 0; i < n; i++) {
        accumulator = accumulator + x[i];
        out[i] = accumulator;
    }
}

/* Segmented form of the loop above: the accumulator starts again at every element whose head flag is
 * non-zero (and at element 0). No reference counterpart (examples/scan.py scans one segment); it is the
 * serial definition the segmented entry point of the library is checked against. */
void oracle_segmented_scan_cpu(size_t n, const uint32_t* x, const uint8_t* heads, uint32_t* out) {
    uint32_t accumulator = 0;
    for (size_t i = 0; i < n; i++) {
        if (heads[i]) accumulator = 0;
        accumulator = accumulator + x[i];
        out[i] = accumulator;
    }
}

/* The loop of scan_cpu (evals/4090_scan/scan_harness.cuh:30-36) on 64-bit elements, modulo 2^64. */
void oracle_scan_i64_cpu(size_t n, const uint64_t* x, uint64_t* out) {
    uint64_t accumulator = 0;
    for (size_t i = 0; i < n; i++) {
        accumulator = accumulator + x[i];
        out[i] = accumulator;
    }
}

/* Exclusive form of the loop above (same accumulator, written before it takes the element in):
 * out[0] = 0, out[i] = x[0] + ... + x[i-1]. No reference counterpart; it is the serial definition
 * the exclusive entry point of the library is checked against. */
void oracle_scan_exclusive_cpu(size_t n, const uint32_t* x, uint32_t* out) {
    uint32_t accumulator = 0;
    for (size_t i = 0; i < n; i++) {
        const uint32_t element = x[i];  /* x may be out */
        out[i] = accumulator;
        accumulator = accumulator + element;
    }
}

/* The same serial loop with a maximum of signed 32-bit integers in place of the sum: out[i] =
 * max(x[0], ..., x[i]). No reference counterpart (the reference scans sums, scan_harness.cuh:30-36); it is
 * the serial definition the running-maximum entry point of the library is checked against. */
void oracle_scan_max_cpu(size_t n, const int32_t* x, int32_t* out) {
    int32_t best = INT32_MIN;
    for (size_t i = 0; i < n; i++) {
        if (x[i] > best) best = x[i];
        out[i] = best;
    }
}

/*
 * Structure-preserving restatement of the GPU algorithm
 * (examples/scan.py:106-227, evals/4090_scan/main.cu:63-86), run serially:
 * blocks of 16384 = 512 rows x 32; each row a Kogge-Stone scan with strides
 * 1,2,4,8,16 (scan_warps); the 512 row ends scanned by 9 Hillis-Steele rounds
 * with ping-pong buffers (naive_scan_warp_ends); block aggregate published;
 * look-back over predecessors summing aggregates until a prefix is met
 * (lookback_to_prev_blocks); write-back adds prefix + previous row total
 * (update_with_new_data_and_writeback). As in the reference launcher only
 * n / 16384 whole blocks are processed, in place; a tail stays untouched.
 * On the GPU the timing of the other blocks decides how far a look-back walks
 * before it meets a published prefix; the result does not depend on it.
 * `stall_every` models that here: with stall_every = s > 0 only blocks whose
 * index is a multiple of s ever show their prefix, so every look-back has to
 * chase up to s-1 aggregates (the else-branch of the reference loop); 0 means
 * every prefix is visible at once (look-back depth 1).
 * Returns the number of blocks processed.
 */
size_t oracle_scan_lookback(size_t n, uint32_t* x, unsigned stall_every) {
    enum { BLOCK = 16384, ROW = 32, ROWS = BLOCK / ROW };
    const size_t blocks = n / BLOCK;
    if (blocks == 0) return 0;
    uint32_t* agg = (uint32_t*)malloc(blocks * sizeof(uint32_t));
    uint32_t* pre = (uint32_t*)malloc(blocks * sizeof(uint32_t));
    unsigned char* pre_ready = (unsigned char*)calloc(blocks, 1);
    uint32_t* sh = (uint32_t*)malloc(BLOCK * sizeof(uint32_t));
    uint32_t ends_a[ROWS], ends_b[ROWS];
    if (!agg || !pre || !pre_ready || !sh) { free(agg); free(pre); free(pre_ready); free(sh); return 0; }

    for (size_t b = 0; b < blocks; ++b) {
        uint32_t* xb = x + b * BLOCK;
        /* scan_warps: per row Kogge-Stone; all lanes read before any writes per stride */
        for (int r = 0; r < ROWS; ++r) {
            uint32_t val[ROW], rec[ROW];
            for (int t = 0; t < ROW; ++t) val[t] = xb[r * ROW + t];
            for (int stride = 1; stride < ROW; stride *= 2) {
                for (int t = 0; t < ROW; ++t) rec[t] = (t >= stride) ? val[t - stride] : val[t];
                for (int t = 0; t < ROW; ++t) if (t >= stride) val[t] = rec[t] + val[t];
            }
            for (int t = 0; t < ROW; ++t) sh[r * ROW + t] = val[t];
        }
        /* get_warp_ends_inclusive */
        for (int r = 0; r < ROWS; ++r) ends_a[r] = sh[r * ROW + ROW - 1];
        /* naive_scan_warp_ends: ping-pong Hillis-Steele */
        uint32_t *cur = ends_a, *buf = ends_b;
        for (int stride = 1; stride < ROWS; stride *= 2) {
            for (int i = 0; i < ROWS; ++i) buf[i] = (i >= stride) ? cur[i] + cur[i - stride] : cur[i];
            uint32_t* tmp = cur; cur = buf; buf = tmp;
        }
        const uint32_t aggregate = cur[ROWS - 1];
        agg[b] = aggregate; /* write_block_aggregate */
        /* lookback_to_prev_blocks */
        uint32_t res = 0;
        for (long long id = (long long)b - 1; id >= 0; --id) {
            if (pre_ready[id]) { res = pre[id] + res; break; }
            res = agg[id] + res;
        }
        /* write_block_prefix (optionally withheld to exercise deep look-back) */
        pre[b] = aggregate + res;
        pre_ready[b] = (stall_every == 0) || (b % stall_every == 0);
        /* update_with_new_data_and_writeback */
        for (int r = 0; r < ROWS; ++r)
            for (int t = 0; t < ROW; ++t)
                xb[r * ROW + t] = (r == 0) ? res + sh[t] : res + cur[r - 1] + sh[r * ROW + t];
    }
    free(agg); free(pre); free(pre_ready); free(sh);
    return blocks;
}

/* ------------------------------------------------------------------ sgemm */

/*
 * C = alpha*A@B + beta*C the way kernels 1-4 compute it
 * (generated/my_sgemm_kernel_1.cu:18-23): per element a serial fp32 sum over
 * increasing k, then alpha*tmp + beta*C. The reference builds with nvcc's
 * default -fmad=true (evals/4090_sgemm/Makefile), i.e. `tmp += a*b` is one
 * fused multiply-add and the final a*x+b*y contracts to fma(alpha,tmp,beta*c);
 * that is written out here with fmaf so the result is defined bit for bit.
 * beta == 0 does not read C (BLAS convention; the library documents it).
 */
void oracle_sgemm_fma(int M, int N, int K, float alpha, const float* A, const float* B, float beta,
                      float* C) {
    for (int i = 0; i < M; ++i) {
        for (int j = 0; j < N; ++j) {
            float tmp = 0.0f;
            for (int k = 0; k < K; ++k) tmp = fmaf(A[(size_t)i * K + k], B[(size_t)k * N + j], tmp);
            float* c = &C[(size_t)i * N + j];
            *c = (beta == 0.0f) ? alpha * tmp : fmaf(alpha, tmp, beta * (*c));
        }
    }
}

/* Same product with every operation in double: the tolerance oracle
 * (max |err| <= 1e-5 * sqrt(K) * max|A| * max|B|). C_in may be NULL when beta == 0. */
void oracle_sgemm_f64(int M, int N, int K, float alpha, const float* A, const float* B, float beta,
                      const float* C_in, double* out) {
    for (int i = 0; i < M; ++i) {
        double* row = out + (size_t)i * N;
        for (int j = 0; j < N; ++j) row[j] = 0.0;
        for (int k = 0; k < K; ++k) {
            const double a = (double)A[(size_t)i * K + k];
            const float* b = B + (size_t)k * N;
            for (int j = 0; j < N; ++j) row[j] += a * (double)b[j];
        }
        for (int j = 0; j < N; ++j) {
            const double ab = (double)alpha * row[j];
            row[j] = (beta == 0.0f) ? ab : ab + (double)beta * (double)C_in[(size_t)i * N + j];
        }
    }
}

/* -------------------------------------------------------------- bf16 gemm */

/* fp32 -> bf16 round-to-nearest-even, the conversion the reference gets from
 * `bf16 = float` assignments (evals/h100_bench/main.cu:36-41, __float2bfloat16_rn). */
uint16_t oracle_f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u); /* NaN */
    return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

float oracle_bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

void oracle_f32_to_bf16_array(const float* src, uint16_t* dst, size_t n) {
    for (size_t i = 0; i < n; ++i) dst[i] = oracle_f32_to_bf16(src[i]);
}

/* D[m][n] = sum_k A[m][k] * B[n][k] in double, A MxK and B NxK row-major bf16
 * (operand layout of examples/h100_matmul.py: both K-contiguous;
 * cuBLAS call evals/h100_bench/main.cu:64-67 computes the same product).
 * D is row-major MxN. */
void oracle_gemm_bf16_f64(int M, int N, int K, const uint16_t* A, const uint16_t* B, double* D) {
    float* bf = (float*)malloc((size_t)(K > 0 ? K : 1) * sizeof(float));
    for (int i = 0; i < M; ++i) {
        for (int k = 0; k < K; ++k) bf[k] = oracle_bf16_to_f32(A[(size_t)i * K + k]);
        for (int j = 0; j < N; ++j) {
            const uint16_t* b = B + (size_t)j * K;
            double s = 0.0;
            for (int k = 0; k < K; ++k) s += (double)bf[k] * (double)oracle_bf16_to_f32(b[k]);
            D[(size_t)i * N + j] = s;
        }
    }
    free(bf);
}
