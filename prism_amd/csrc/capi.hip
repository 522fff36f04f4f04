// extern "C" surface of libprism_amd.so; declarations and the reference
// interfaces they replace are in include/prism_amd.h.
#include "../../include/prism_amd.h"

#include <cstring>

#include "common.h"
#include "tile_map.h"

namespace prism {
char* error_buffer() {
    static thread_local char buf[kErrorBufferLen] = {0};
    return buf;
}
}  // namespace prism

using namespace prism;

extern "C" {

const char* prism_version(void) { return "0.1.0"; }

const char* prism_last_error_string(void) { return error_buffer(); }

int prism_device_info(int* cu_count, int* clock_khz, int* wavefront_size, size_t* lds_bytes,
                      size_t* hbm_bytes, char* name, size_t name_len) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
    hipDeviceProp_t p;
    e = hipGetDeviceProperties(&p, dev);
    if (e != hipSuccess) return hip_fail(e, "hipGetDeviceProperties");
    if (cu_count) *cu_count = p.multiProcessorCount;
    if (clock_khz) *clock_khz = p.clockRate;
    if (wavefront_size) *wavefront_size = p.warpSize;
    if (lds_bytes) *lds_bytes = p.sharedMemPerBlock;
    if (hbm_bytes) *hbm_bytes = p.totalGlobalMem;
    if (name && name_len) {
        strncpy(name, p.gcnArchName, name_len - 1);
        name[name_len - 1] = 0;
    }
    return 0;
}

int prism_tile_coords(int workgroup_id, int tiles_m, int tiles_n, int* tile_m, int* tile_n) {
    if (tiles_m <= 0 || tiles_n <= 0 || workgroup_id < 0 ||
        static_cast<long long>(workgroup_id) >= static_cast<long long>(tiles_m) * tiles_n)
        return fail(1, "prism_tile_coords: id %d outside a %d x %d tile grid", workgroup_id, tiles_m, tiles_n);
    if (!tile_m || !tile_n) return fail(1, "prism_tile_coords: null output");
    xcd_tile_coords(workgroup_id, tiles_m, tiles_n, *tile_m, *tile_n);
    return 0;
}

int prism_wave_regroup_i32(const int32_t* in, int32_t* out, size_t n, int items_per_lane, int direction, void* stream) {
    return launch_wave_regroup(in, out, n, items_per_lane, direction, static_cast<hipStream_t>(stream));
}

int prism_add_m(const int32_t* x, int32_t* y, int32_t m, size_t n, void* stream) {
    return launch_add_m(x, y, m, n, static_cast<hipStream_t>(stream));
}

size_t prism_scan_workspace_bytes(size_t n) { return scan_workspace_bytes(n); }

static_assert(PRISM_SCAN_EXCLUSIVE == kFlagExclusive && PRISM_SCAN_TICKET_ORDER == kFlagTicket &&
                  PRISM_SCAN_NO_HELP == kFlagNoHelp && PRISM_SCAN_OP_MAX == kFlagOpMax && PRISM_SCAN_OP_MIN == kFlagOpMin &&
                  PRISM_ERROR_SCAN_ORDER == kScanOrderError && PRISM_ERROR_SCAN_WORKSPACE == kScanWorkspaceError,
              "include/prism_amd.h and common.h disagree");

static const uint32_t* u32(const int32_t* p) { return reinterpret_cast<const uint32_t*>(p); }
static uint32_t* u32(int32_t* p) { return reinterpret_cast<uint32_t*>(p); }

int prism_scan_workspace_init(void* workspace, size_t workspace_bytes, void* stream) {
    return scan_workspace_init(workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

int prism_scan_status(void* workspace, size_t workspace_bytes, void* stream) {
    return scan_status(workspace, workspace_bytes, static_cast<hipStream_t>(stream));
}

int prism_scan_i32(const int32_t* in, int32_t* out, size_t n, void* workspace,
                   size_t workspace_bytes, void* stream) {
    return launch_scan(u32(in), u32(out), n, workspace, workspace_bytes, 0u, -1, static_cast<hipStream_t>(stream));
}

int prism_scan_i32_ex(const int32_t* in, int32_t* out, size_t n, void* workspace, size_t workspace_bytes,
                      unsigned flags, long long spin_limit, void* stream) {
    return launch_scan(u32(in), u32(out), n, workspace, workspace_bytes, flags, spin_limit,
                       static_cast<hipStream_t>(stream));
}

int prism_scan_i32_static(const int32_t* in, int32_t* out, size_t n, void* stream) {
    return launch_scan_static(u32(in), u32(out), n, static_cast<hipStream_t>(stream));
}

int prism_scan_exclusive_i32(const int32_t* in, int32_t* out, size_t n, void* workspace,
                             size_t workspace_bytes, void* stream) {
    return launch_scan(u32(in), u32(out), n, workspace, workspace_bytes, kFlagExclusive, -1,
                       static_cast<hipStream_t>(stream));
}

int prism_scan_max_i32(const int32_t* in, int32_t* out, size_t n, void* workspace,
                       size_t workspace_bytes, void* stream) {
    return launch_scan(u32(in), u32(out), n, workspace, workspace_bytes, kFlagOpMax, -1,
                       static_cast<hipStream_t>(stream));
}

int prism_scan_min_i32(const int32_t* in, int32_t* out, size_t n, void* workspace,
                       size_t workspace_bytes, void* stream) {
    return launch_scan(u32(in), u32(out), n, workspace, workspace_bytes, kFlagOpMin, -1,
                       static_cast<hipStream_t>(stream));
}

int prism_segmented_scan_i32(const int32_t* in, const uint8_t* heads, int32_t* out, size_t n, void* workspace,
                             size_t workspace_bytes, void* stream) {
    return launch_segmented_scan(u32(in), heads, u32(out), n, workspace, workspace_bytes, 0u, -1, static_cast<hipStream_t>(stream));
}

int prism_segmented_scan_i32_ex(const int32_t* in, const uint8_t* heads, int32_t* out, size_t n, void* workspace,
                                size_t workspace_bytes, unsigned flags, long long spin_limit, void* stream) {
    return launch_segmented_scan(u32(in), heads, u32(out), n, workspace, workspace_bytes, flags, spin_limit,
                                 static_cast<hipStream_t>(stream));
}

int prism_scan_i64(const int64_t* in, int64_t* out, size_t n, void* workspace, size_t workspace_bytes, void* stream) {
    return launch_scan64(reinterpret_cast<const unsigned long long*>(in), reinterpret_cast<unsigned long long*>(out), n,
                         workspace, workspace_bytes, 0u, -1, static_cast<hipStream_t>(stream));
}

int prism_scan_i64_ex(const int64_t* in, int64_t* out, size_t n, void* workspace, size_t workspace_bytes, unsigned flags,
                      long long spin_limit, void* stream) {
    return launch_scan64(reinterpret_cast<const unsigned long long*>(in), reinterpret_cast<unsigned long long*>(out), n,
                         workspace, workspace_bytes, flags, spin_limit, static_cast<hipStream_t>(stream));
}

uint32_t* prism_launch_scan(size_t n, uint32_t* x, void* workspace) {
    // The reference's launcher accepts any workspace contents (it clears them itself,
    // evals/4090_scan/main.cu:81-82), so this one initialises before every scan.
    if (n == 0) return x;
    if (scan_workspace_init(workspace, scan_workspace_bytes(n), nullptr) != 0) return nullptr;
    int rc = launch_scan(x, x, n, workspace, scan_workspace_bytes(n), 0u, -1, nullptr);
    return rc == 0 ? x : nullptr;
}

int prism_sgemm(int variant, int M, int N, int K, float alpha, const float* A, const float* B,
                float beta, float* C, void* stream) {
    return launch_sgemm(variant, M, N, K, alpha, A, B, beta, C, static_cast<hipStream_t>(stream));
}

size_t prism_sgemm_workspace_bytes(int M, int N, int K) { return sgemm_workspace_bytes(M, N, K); }

int prism_sgemm_ws(int variant, int M, int N, int K, float alpha, const float* A, const float* B, float beta,
                   float* C, void* workspace, size_t workspace_bytes, void* stream) {
    return launch_sgemm_ws(variant, M, N, K, alpha, A, B, beta, C, workspace, workspace_bytes,
                           static_cast<hipStream_t>(stream));
}

int prism_sgemm_ws_plan(int M, int N, int K, size_t workspace_bytes, int* workgroups, int* shared_tiles) {
    return sgemm_ws_plan(M, N, K, workspace_bytes, workgroups, shared_tiles);
}

int prism_run_my_kernel(int my_kernel_num, int M, int N, int K, float alpha, float* A, float* B,
                        float beta, float* C) {
    if (my_kernel_num < 1 || my_kernel_num > 5)
        return fail(1, "Unknown my_kernel number %d (expected 1..5)", my_kernel_num);
    return launch_sgemm(my_kernel_num, M, N, K, alpha, A, B, beta, C, nullptr);
}

int prism_gemm_bf16(int M, int N, int K, const uint16_t* A, const uint16_t* B, float* D,
                    void* stream) {
    return launch_gemm_bf16(M, N, K, A, B, D, nullptr, static_cast<hipStream_t>(stream));
}

int prism_runmyh100(int M, int N, int K, const uint16_t* A, const uint16_t* B, uint16_t* C,
                    int* DB) {
    (void)DB;
    return launch_gemm_bf16(M, N, K, A, B, nullptr, C, nullptr);
}

}  // extern "C"
