// Shared host-side helpers for libprism_amd.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstddef>
#include <cstdint>
#include <cstdio>

namespace prism {

constexpr int kWave = 64;  // CDNA wavefront width; every kernel here assumes it

// Thread-local error text behind prism_last_error_string().
char* error_buffer();
constexpr size_t kErrorBufferLen = 512;

inline int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(error_buffer(), kErrorBufferLen, fmt, ap);
    va_end(ap);
    return code;
}

inline int hip_fail(hipError_t e, const char* what) {
    return fail(static_cast<int>(e), "%s: %s", what, hipGetErrorString(e));
}

// Launch check: hipGetLastError() clears and returns the launch error, if any.
inline int check_launch(const char* kernel) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return hip_fail(e, kernel);
    return 0;
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline bool aligned4(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 3u) == 0; }
inline bool aligned2(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 1u) == 0; }

template <typename T>
constexpr T ceil_div(T a, T b) { return (a + b - 1) / b; }

// Compute units of the current device (the launchers size their tile choices by it).
inline int cu_count() {
    static int cached[64] = {};  // per device; a racing first call writes the same value
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cached[dev] == 0) {
        int cus = 0;
        if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) cus = 256;
        cached[dev] = cus;
    }
    return cached[dev];
}

// Internal launchers, one per kernel family (defined in the .hip files).
int launch_add_m(const int32_t* x, int32_t* y, int32_t m, size_t n, hipStream_t s);
// Scan flags and error code: the values of PRISM_SCAN_* / PRISM_ERROR_SCAN_ORDER in include/prism_amd.h.
constexpr unsigned kFlagExclusive = 1u, kFlagTicket = 2u, kFlagNoHelp = 4u;
constexpr unsigned kFlagOpMask = 0x30u, kFlagOpSum = 0x00u, kFlagOpMax = 0x10u, kFlagOpMin = 0x20u;
constexpr int kScanOrderError = 10001, kScanWorkspaceError = 10002;
size_t scan_workspace_bytes(size_t n);
int scan_workspace_init(void* ws, size_t ws_bytes, hipStream_t s);
// spin_limit < 0: the library's bound on the polls of a look-back window; 0: a look-back never waits.
int launch_scan(const uint32_t* in, uint32_t* out, size_t n, void* ws, size_t ws_bytes, unsigned flags,
                long long spin_limit, hipStream_t s);
int scan_status(void* ws, size_t ws_bytes, hipStream_t s);
// flags: kFlagNoHelp or 0; spin_limit as for launch_scan.
int launch_segmented_scan(const uint32_t* in, const uint8_t* heads, uint32_t* out, size_t n, void* ws, size_t ws_bytes,
                          unsigned flags, long long spin_limit, hipStream_t s);
int launch_scan64(const unsigned long long* in, unsigned long long* out, size_t n, void* ws, size_t ws_bytes, unsigned flags,
                  long long spin_limit, hipStream_t s);
int launch_scan_static(const uint32_t* in, uint32_t* out, size_t n, hipStream_t s);
int launch_wave_regroup(const int32_t* in, int32_t* out, size_t n, int items_per_lane, int direction, hipStream_t s);
int launch_sgemm(int variant, int M, int N, int K, float alpha, const float* A, const float* B,
                 float beta, float* C, hipStream_t s);
// 0 if the arguments are ones launch_sgemm accepts, else the error (and the error string is set).
int check_sgemm_arguments(int variant, int M, int N, int K, const float* A, const float* B, const float* C);
size_t sgemm_workspace_bytes(int M, int N, int K);
// What launch_sgemm_ws does for this shape with 16 B-aligned operands and ws_bytes of workspace: the number of
// workgroups that share K ranges and of the tiles they share (both 0: the call is launch_sgemm).
int sgemm_ws_plan(int M, int N, int K, size_t ws_bytes, int* groups, int* sk_tiles);
int launch_sgemm_ws(int variant, int M, int N, int K, float alpha, const float* A, const float* B, float beta,
                    float* C, void* ws, size_t ws_bytes, hipStream_t s);
int launch_gemm_bf16(int M, int N, int K, const uint16_t* A, const uint16_t* B, float* D_f32,
                     uint16_t* C_bf16_colmajor, hipStream_t s);

}  // namespace prism
