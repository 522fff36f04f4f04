/*
 * prism_amd.h - C ABI of libprism_amd.so: the MI355X (gfx950) kernels behind the
 * host launchers of manya-bansal/prism's evaluation harnesses.
 *
 * Conventions shared by every entry point
 *   - All data pointers are DEVICE pointers owned by the caller (a raw
 *     hipMalloc pointer, or tensor.data_ptr() of a PyTorch-ROCm tensor).
 *   - `stream` is a hipStream_t passed as void*; NULL means the default stream.
 *   - Calls are asynchronous: they enqueue work and return. The caller
 *     synchronises, as the reference harnesses do after their launchers.
 *   - Functions returning int return 0 on success, otherwise a non-zero
 *     hipError_t value (1 = invalid argument); prism_last_error_string() then
 *     describes the failure for the calling thread.
 *   - No entry point reads the environment or keeps options between calls
 *     (every choice is an argument), so all of them are re-entrant and may be
 *     used from several host threads.
 *
 * "Reference" citations below are paths in the manya-bansal/prism tree.
 */
#ifndef PRISM_AMD_H
#define PRISM_AMD_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------ misc -- */

/* Library version, "major.minor.patch". */
const char* prism_version(void);

/* Message for the last failure on the calling thread ("" if none). */
const char* prism_last_error_string(void);

/*
 * Properties of the current HIP device, for the roofline report. Any pointer
 * may be NULL. clock_khz is the device's peak engine clock, lds_bytes the LDS
 * available to one workgroup, hbm_bytes the total device memory.
 */
int prism_device_info(int* cu_count, int* clock_khz, int* wavefront_size,
                      size_t* lds_bytes, size_t* hbm_bytes, char* name,
                      size_t name_len);

/*
 * Host-side evaluation of the workgroup-id -> output-tile map the two MFMA
 * GEMM kernels use (the role of Schedule, evals/h100_bench/utils.cuh:277-307,
 * redone for 8 XCDs). Runs on the CPU; lets a caller or test check that the map
 * visits every tile of a tiles_m x tiles_n grid exactly once.
 */
int prism_tile_coords(int workgroup_id, int tiles_m, int tiles_n, int* tile_m, int* tile_n);

/* ----------------------------------------------------------------- add_m -- */

/*
 * y[i] = x[i] + m for i in [0, n), int32 with two's-complement wrap-around.
 * Replaces the kernel Prism emits for `add_m_thread`
 * (examples/add_m_thread.py:10-19, generated text README.md:133-140), whose
 * signature is add_m(x, y, m) with one thread per element and no bound; here
 * the element count is explicit. x == y is allowed.
 */
int prism_add_m(const int32_t* x, int32_t* y, int32_t m, size_t n, void* stream);

/*
 * The reference's warp_load / warp_store (examples/warp_load.py:13-22,
 * warp_store.py:13-22, with thread_load.py / thread_store.py) as an operator on
 * 64-lane wavefronts: every chunk of 64 * items_per_lane ints is moved between
 * the arrangement those functions give a warp (lane l holds items
 * [l * items_per_lane, (l + 1) * items_per_lane), "blocked") and the one in
 * which every instruction of the wavefront touches 64 consecutive ints
 * ("striped": item j of lane l is element 64 j + l).
 *   direction 0: out[c][64 j + l] = in[c][items_per_lane * l + j]
 *   direction 1: the inverse
 * for chunk c. items_per_lane is 1, 2, 4, 8 or 16; any n (a last, partial
 * chunk counts as one padded with zeros: positions at or beyond n are neither
 * read nor written, every position below n is written); in and out must not
 * overlap.
 */
int prism_wave_regroup_i32(const int32_t* in, int32_t* out, size_t n, int items_per_lane,
                           int direction, void* stream);

/* ------------------------------------------------------------------ scan -- */

/*
 * Bytes of device workspace the scans need for n elements: a 256-byte header
 * and 16 bytes per 16384 elements plus 16 (the size the reference's launcher
 * uses, n / 16384 * 16 + 4, rounded up). Replaces scan_gpu::get_workspace_size
 * (evals/4090_scan/main.cu:63-66). Never 0, so a caller may always allocate it.
 * A workspace sized for n serves every smaller n too.
 */
size_t prism_scan_workspace_bytes(size_t n);

/*
 * Brings a workspace (16-byte aligned) into its initial state (zeros and a
 * magic word in the header). Call it once after allocating; a scan on a
 * workspace without the magic word touches nothing in it and
 * prism_scan_status reports PRISM_ERROR_SCAN_WORKSPACE.
 * The reference clears its workspace with two cudaMemset calls in front of
 * every launch (evals/4090_scan/main.cu:81-82); here every scan leaves the
 * workspace ready for the next one, so no clearing launch sits in front of a
 * scan. Enqueues a fill kernel on `stream` (no memset node, so the call can be
 * captured into a HIP graph).
 */
int prism_scan_workspace_init(void* workspace, size_t workspace_bytes, void* stream);

/*
 * Inclusive prefix sum, out[i] = in[0] + ... + in[i] modulo 2^32 (identical
 * bit patterns for int32 and uint32). Single pass with decoupled look-back
 * between tiles. Any n >= 0; in == out is allowed (in-place, as the reference
 * runs); partial overlap is not. The workspace must be initialised (above) and
 * hold prism_scan_workspace_bytes(n) bytes; calls that share a workspace must
 * be ordered on one stream, and may differ in n and in kind.
 * Tiles are numbered by workgroup id, which waits least when workgroups start
 * in id order (prism_scan_i32_ex can select the reference's ticket counter
 * instead), but the result does not rest on that order: a tile whose
 * predecessor stays silent for milliseconds forms that predecessor's sum from
 * the input itself, so every tile finishes on its own and the sums are the
 * same bits however the workgroups were started. A return value of 0 means the
 * call was enqueued; what can still invalidate the output is a workspace that
 * was never initialised, which prism_scan_status reports once the stream has
 * drained.
 * Replaces scan_kernel + its device helpers (examples/scan.py:23-227,
 * generated/scan_kernel.cu:1-29).
 */
int prism_scan_i32(const int32_t* in, int32_t* out, size_t n, void* workspace,
                   size_t workspace_bytes, void* stream);

/* Flags of prism_scan_i32_ex (one PRISM_SCAN_OP_* value, or-ed with the others). */
enum {
    PRISM_SCAN_EXCLUSIVE = 1,     /* prism_scan_exclusive_i32's result                                  */
    PRISM_SCAN_TICKET_ORDER = 2,  /* tiles numbered by get_block_idx_from_global_counter's ticket        */
                                  /* (examples/scan.py:88-99) instead of by workgroup id                 */
    PRISM_SCAN_NO_HELP = 4,       /* a look-back that runs out of polls reports it (prism_scan_status)   */
                                  /* and goes on with a wrong sum instead of helping its predecessor:    */
                                  /* the plain bounded wait, kept to exercise that way out (every kind   */
                                  /* of scan takes this flag through its _ex entry point)                */
    PRISM_SCAN_OP_SUM = 0x00,
    PRISM_SCAN_OP_MAX = 0x10,     /* prism_scan_max_i32's result (inclusive, workgroup-id order only)    */
    PRISM_SCAN_OP_MIN = 0x20      /* prism_scan_min_i32's result (inclusive, workgroup-id order only)    */
};

/* prism_scan_status: a tile gave up waiting for its predecessors. */
#define PRISM_ERROR_SCAN_ORDER 10001
/* prism_scan_status: the workspace was never initialised (or was overwritten). */
#define PRISM_ERROR_SCAN_WORKSPACE 10002

/*
 * prism_scan_i32 with every choice spelled out as an argument (the library
 * reads no environment variables and keeps no options between calls).
 * spin_limit bounds the polls of one look-back window before the tile stops
 * waiting for a silent predecessor and helps it (forms its sum from the
 * input), or, with PRISM_SCAN_NO_HELP, reports and goes on: negative = the
 * library's default (2^12 polls, milliseconds; 2^22 with PRISM_SCAN_NO_HELP),
 * 0 = no waiting at all, which exercises either way out from the host without
 * a stuck predecessor. The reference's kernel waits without bound
 * (generated/lookback_to_prev_blocks.cu:12-21).
 */
int prism_scan_i32_ex(const int32_t* in, int32_t* out, size_t n, void* workspace,
                      size_t workspace_bytes, unsigned flags, long long spin_limit,
                      void* stream);

/*
 * prism_scan_i32 without a workspace argument and without any allocation: the
 * status words live in a device array that is part of the library (2 MiB + 256
 * bytes per GPU, held until the process ends), so n is limited to 2^31
 * elements; a larger n returns 1 with an error string. No counterpart in the
 * reference. It is for callers that cannot allocate: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc. The call makes
 * no hipMalloc / hipFree and uses no allocating library routine. The first call
 * on a device looks the array's address up and fills it once; that call must
 * be made outside stream capture (prism_scan_status(NULL, 0, stream) serves as
 * well), later ones may be captured. All calls on one GPU share that GPU's
 * array: they must be ordered on one stream, calls that overlap on one GPU
 * race. Same kernels and same result as prism_scan_i32;
 * prism_scan_status(NULL, 0, stream) reports for the library's array.
 */
int prism_scan_i32_static(const int32_t* in, int32_t* out, size_t n, void* stream);

/*
 * Waits for `stream`, then reports on the scans that used this workspace
 * since the last report: 0 = nothing to report; PRISM_ERROR_SCAN_WORKSPACE =
 * the workspace was not initialised (or something else wrote into it);
 * PRISM_ERROR_SCAN_ORDER = a look-back gave up waiting (only scans that were
 * told not to help, PRISM_SCAN_NO_HELP). In both cases
 * the output of those scans is invalid, the error string says more, and the
 * workspace has been initialised afresh.
 * workspace == NULL stands for the array prism_scan_i32_static uses on the
 * current device. The reference has no counterpart (its look-back cannot give up); this is what
 * turns a broken tile-order assumption into an error instead of a wrong sum.
 */
int prism_scan_status(void* workspace, size_t workspace_bytes, void* stream);

/*
 * Exclusive prefix sum, out[i] = in[0] + ... + in[i-1] modulo 2^32, out[0] = 0: the same single-pass
 * kernel with a different write-back stage (the stage of update_with_new_data_and_writeback,
 * examples/scan.py:174-193). Arguments, workspace and aliasing rules as for prism_scan_i32. The
 * reference's harness only times inclusive sums (evals/4090_scan/bench.cu:96-116); this form is what
 * callers that turn counts into offsets need.
 */
int prism_scan_exclusive_i32(const int32_t* in, int32_t* out, size_t n, void* workspace,
                             size_t workspace_bytes, void* stream);

/*
 * Running maximum of signed 32-bit integers, out[i] = max(in[0], ..., in[i]): the same single-pass kernel
 * with the addition of scan_kernel's stages (examples/scan.py:106-173, the combination of aggregates in
 * lookback_to_prev_blocks :34-85) replaced by a maximum and 0 by INT32_MIN. Arguments, workspace and
 * aliasing rules as for prism_scan_i32; tiles are always numbered by workgroup id. The reference scans
 * sums only; this is the operator form of the same decomposition.
 */
int prism_scan_max_i32(const int32_t* in, int32_t* out, size_t n, void* workspace,
                       size_t workspace_bytes, void* stream);

/*
 * Running minimum, out[i] = min(in[0], ..., in[i]): prism_scan_max_i32 with the order reversed (the
 * operator form of examples/scan.py:106-173 again, identity INT32_MAX).
 */
int prism_scan_min_i32(const int32_t* in, int32_t* out, size_t n, void* workspace,
                       size_t workspace_bytes, void* stream);

/*
 * Segmented inclusive prefix sum: out[i] = the sum of in[j] over j from the last
 * element at or before i whose byte in `heads` is non-zero (element 0 always
 * starts a segment) up to i, modulo 2^32. The same single pass with the sum of
 * scan_kernel's stages (examples/scan.py:106-227; the combination of records in
 * lookback_to_prev_blocks :60-85) replaced by the associative, non-commutative
 * operator on (head seen, sum) pairs; a tile's walk back ends at the nearest
 * tile that holds a head. Workspace, aliasing of in and out, ordering and the
 * status check as for prism_scan_i32; heads must not overlap out. The reference
 * scans one segment only.
 */
int prism_segmented_scan_i32(const int32_t* in, const uint8_t* heads, int32_t* out, size_t n,
                             void* workspace, size_t workspace_bytes, void* stream);

/*
 * prism_segmented_scan_i32 with the look-back's choices as arguments, as
 * prism_scan_i32_ex has them: flags is 0 or PRISM_SCAN_NO_HELP, spin_limit the
 * bound on the polls of one look-back window (negative = the library's
 * default, 0 = no waiting). A tile that helps forms its predecessor's (head
 * seen, sum) pair from that tile's input and head bytes. The reference's
 * look-back waits without bound (generated/lookback_to_prev_blocks.cu:12-21).
 */
int prism_segmented_scan_i32_ex(const int32_t* in, const uint8_t* heads, int32_t* out, size_t n,
                                void* workspace, size_t workspace_bytes, unsigned flags,
                                long long spin_limit, void* stream);

/*
 * Inclusive prefix sum of 64-bit elements, out[i] = in[0] + ... + in[i] modulo
 * 2^64 (identical bit patterns for int64 and uint64): scan_kernel's
 * decomposition (examples/scan.py:106-227) on wider elements. A tile publishes
 * its 64-bit aggregate and prefix as two status words (state + half each) and
 * a reader accepts them only as a pair of the same state. Pointers 8-byte
 * aligned (16-byte aligned ones take the fast path); workspace
 * (prism_scan_workspace_bytes(n) for the same n), aliasing, ordering and the
 * status check as for prism_scan_i32. The reference scans uint32 only
 * (evals/4090_scan/scan_harness.cuh:30-36).
 */
int prism_scan_i64(const int64_t* in, int64_t* out, size_t n, void* workspace,
                   size_t workspace_bytes, void* stream);

/*
 * prism_scan_i64 with the look-back's choices as arguments (flags 0 or
 * PRISM_SCAN_NO_HELP, spin_limit as for prism_scan_i32_ex). The reference's
 * look-back waits without bound (generated/lookback_to_prev_blocks.cu:12-21).
 */
int prism_scan_i64_ex(const int64_t* in, int64_t* out, size_t n, void* workspace,
                      size_t workspace_bytes, unsigned flags, long long spin_limit,
                      void* stream);

/*
 * The reference launcher's own shape: in-place on x, default stream, returns
 * the device pointer that holds the result (x) or NULL on failure.
 * Replaces scan_gpu::launch_scan (evals/4090_scan/main.cu:68-86). Like the
 * reference it accepts a workspace with any contents and clears it inside the
 * call. Unlike the reference, n need not be a multiple of 16384. The workspace
 * must hold at least prism_scan_workspace_bytes(n) bytes.
 */
uint32_t* prism_launch_scan(size_t n, uint32_t* x, void* workspace);

/* ----------------------------------------------------------------- sgemm -- */

/* Kernel numbers accepted by prism_sgemm / prism_run_my_kernel. */
enum {
    PRISM_SGEMM_BEST = 0,             /* alias of PRISM_SGEMM_WAVE_TILE                        */
    PRISM_SGEMM_NAIVE = 1,            /* my_sgemm_kernel_1: one thread per C element            */
    PRISM_SGEMM_COALESCED = 2,        /* my_sgemm_kernel_2: 32x32 tile thread remap             */
    PRISM_SGEMM_LDS_BLOCK = 3,        /* sgemm_shared_mem_block<32> (the eval's "kernel 3")     */
    PRISM_SGEMM_THREAD_TILE = 4,      /* my_sgemm_kernel_4: 8x8 thread tile, vector loads       */
    PRISM_SGEMM_WAVE_TILE = 5,        /* my_sgemm_kernel_5: wave tile, here on fp32 MFMA        */
    PRISM_SGEMM_THREAD_TILE_SCALAR = 6 /* my_sgemm_kernel_3: 8x8 thread tile, scalar staging     */
};

/*
 * C = alpha * A @ B + beta * C, fp32, row-major, A is MxK, B is KxN, C is MxN,
 * any M, N, K >= 0. When beta == 0, C is never read (NaN/Inf in it do not
 * propagate). `variant` selects the kernel (enum above).
 * Replaces run_my_sgemm_1..5 (evals/4090_sgemm/runner.cu:135-243) and the
 * kernels they launch (generated/my_sgemm_kernel_{1,2,3,4,5}.cu,
 * generated/sgemm_shared_mem_block.cu, evals/4090_sgemm/my_kernel_utils.cuh:13-90).
 */
int prism_sgemm(int variant, int M, int N, int K, float alpha, const float* A,
                const float* B, float beta, float* C, void* stream);

/*
 * prism_sgemm with a workspace. Kernel 5 gives every workgroup one whole output
 * tile, as the reference's launcher does (evals/4090_sgemm/runner.cu:191-243),
 * so a problem whose tiles are not a whole number of rounds of the GPU's compute
 * units leaves most of them idle in the last round, and a skinny problem (few
 * tiles, long K: 128 x 4096 x 4096) leaves them idle throughout. With a
 * workspace the K ranges of the tiles of the last, partial round (of all tiles,
 * when there are fewer than compute units or the problem is skinny) are shared
 * evenly between all compute units: a workgroup that gets part of a tile's K
 * range stores its partial product into the workspace, and a second kernel adds
 * a tile's partial products in the order of k (the same bits on every run on
 * one device) and applies alpha and beta. No workgroup waits for another.
 * prism_sgemm_workspace_bytes says how much a shape can use on the CURRENT
 * device (0: nothing would be shared); query it with the device current that
 * the call will run on. With a smaller or NULL workspace, one that is not
 * 16-byte aligned, operands that are not 16-byte aligned, N or K not a multiple
 * of 4, or any other kernel number, the call is prism_sgemm. Arguments are
 * checked as in prism_sgemm. Calls that share a workspace must be ordered on one
 * stream. No counterpart in the reference, whose launchers take no workspace; a
 * harness that wants the sharing holds one buffer and passes it here.
 */
size_t prism_sgemm_workspace_bytes(int M, int N, int K);
int prism_sgemm_ws(int variant, int M, int N, int K, float alpha, const float* A,
                   const float* B, float beta, float* C, void* workspace,
                   size_t workspace_bytes, void* stream);

/*
 * What prism_sgemm_ws does for this shape on the current device, given 16-byte
 * aligned operands and workspace_bytes of workspace: *workgroups = the number
 * of workgroups that share K ranges, *shared_tiles = the tiles they share
 * (256 x 256 ones, or 64 x 256 for skinny shapes); both 0 when the call would
 * be prism_sgemm. Either pointer may be NULL. Lets a harness or test assert
 * that the workspace path is the one it measures. No counterpart in the
 * reference.
 */
int prism_sgemm_ws_plan(int M, int N, int K, size_t workspace_bytes, int* workgroups,
                        int* shared_tiles);

/*
 * The reference dispatcher's own shape: default stream, kernel numbers 1..5.
 * Replaces run_my_kernel (evals/4090_sgemm/runner.cuh:28-29,
 * runner.cu:245-267). The reference throws std::invalid_argument for an
 * unknown number; this returns 1 and sets the error string.
 */
int prism_run_my_kernel(int my_kernel_num, int M, int N, int K, float alpha,
                        float* A, float* B, float beta, float* C);

/* ------------------------------------------------------------- bf16 gemm -- */

/*
 * D = A @ B^T with bf16 inputs and fp32 accumulation on MFMA.
 * A is MxK row-major bf16, B is NxK row-major bf16 (both K-contiguous, the
 * operand layout of the reference's h100_matmul), D is MxN row-major fp32.
 * Any M, N, K >= 0 (no K tail is dropped). bf16 values are passed as their
 * 16-bit patterns.
 * Replaces cutlass_my_h100_match_no_tail (examples/h100_matmul.py:20-297,
 * generated/cutlass_my_h100_match_no_tail.cu:1-370) with an fp32 result.
 */
int prism_gemm_bf16(int M, int N, int K, const uint16_t* A, const uint16_t* B,
                    float* D, void* stream);

/*
 * The reference launcher's own shape and output layout: C is bf16,
 * COLUMN-major MxN (element (m, n) at C[n * M + m],
 * generated/cutlass_my_h100_match_no_tail.cu:313,347-354), fp32 accumulators
 * rounded to bf16 (round-to-nearest-even) on store; default stream; DB is
 * unused, as in the reference. Replaces prism_h100::runmyh100
 * (evals/h100_bench/utils.cuh:504-533). Holds no cached state, so unlike the
 * reference it may be called with changing shapes and pointers.
 */
int prism_runmyh100(int M, int N, int K, const uint16_t* A, const uint16_t* B,
                    uint16_t* C, int* DB);

#ifdef __cplusplus
}
#endif
#endif /* PRISM_AMD_H */
