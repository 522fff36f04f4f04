// A stand-in for the three harness mains of the reference (evals/4090_scan/main.cu + scan_harness.cuh:112-168,
// evals/4090_sgemm/main.cu:84-147, evals/h100_bench/main.cu:112-141), reduced to their correctness runs, around
// the launcher replacements that the integration guide shows. The test that builds this file extracts those code
// blocks from the guide into integration_snippets.inc, so the text a maintainer would paste is the text compiled,
// linked against libprism_amd.so and run here. Host code only: device memory comes from the HIP runtime API.
#include <hip/hip_runtime_api.h>

#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <stdexcept>
#include <vector>

typedef uint16_t bf16;  // the harness's 16-bit storage type (the reference: __nv_bfloat16)

#include "integration_snippets.inc"

#define HIP_OK(x)                                                                         \
    do {                                                                                  \
        hipError_t e_ = (x);                                                              \
        if (e_ != hipSuccess) {                                                           \
            fprintf(stderr, "%s:%d: %s\n", __FILE__, __LINE__, hipGetErrorString(e_));   \
            exit(2);                                                                      \
        }                                                                                 \
    } while (0)

static uint32_t lcg(uint32_t& s) { return s = s * 1664525u + 1013904223u; }

static uint16_t to_bf16(float f) {  // round to nearest even
    uint32_t u;
    memcpy(&u, &f, 4);
    return static_cast<uint16_t>((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}
static float from_bf16(uint16_t h) {
    uint32_t u = static_cast<uint32_t>(h) << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

// scan_harness.cuh:112-168 in outline: workspace from get_workspace_size, launch, sync, compare with the serial sum.
static int check_scan(size_t n) {
    std::vector<uint32_t> x(n), want(n);
    uint32_t seed = static_cast<uint32_t>(n), acc = 0;
    for (size_t i = 0; i < n; ++i) {
        x[i] = lcg(seed) % 101u;  // U{0..100}, scan_harness.cuh:172
        acc += x[i];
        want[i] = acc;
    }
    uint32_t* dx = nullptr;
    void* ws = nullptr;
    const size_t ws_bytes = scan_gpu::get_workspace_size(n);
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&dx), n * 4));
    HIP_OK(hipMalloc(&ws, ws_bytes));
    HIP_OK(hipMemset(ws, 0xAB, ws_bytes));  // the launcher must not depend on what the workspace holds
    HIP_OK(hipMemcpy(dx, x.data(), n * 4, hipMemcpyHostToDevice));
    uint32_t* out = scan_gpu::launch_scan(n, dx, ws);
    if (out == nullptr) { fprintf(stderr, "scan n=%zu: launcher returned nullptr\n", n); return 1; }
    HIP_OK(hipDeviceSynchronize());
    HIP_OK(hipGetLastError());
    std::vector<uint32_t> got(n);
    HIP_OK(hipMemcpy(got.data(), out, n * 4, hipMemcpyDeviceToHost));
    HIP_OK(hipFree(dx));
    HIP_OK(hipFree(ws));
    for (size_t i = 0; i < n; ++i)
        if (got[i] != want[i]) { fprintf(stderr, "scan n=%zu: mismatch at %zu\n", n, i); return 1; }
    printf("scan n=%zu ok\n", n);
    return 0;
}

// evals/4090_sgemm/main.cu:84-147 in outline: every kernel number against a host product, |d| <= 0.01 (runner.cu:110).
static int check_sgemm(int n) {
    std::vector<float> A(n * n), B(n * n), C(n * n);
    uint32_t seed = 7;
    for (auto* m : {&A, &B, &C})
        for (auto& v : *m) v = static_cast<float>(lcg(seed) % 5u) + 0.01f * static_cast<float>(lcg(seed) % 5u);  // runner.cu:54-65
    const float alpha = 0.5f, beta = 3.0f;  // main.cu:48
    std::vector<double> want(n * n);
    for (int i = 0; i < n; ++i)
        for (int j = 0; j < n; ++j) {
            double s = 0;
            for (int k = 0; k < n; ++k) s += static_cast<double>(A[i * n + k]) * B[k * n + j];
            want[i * n + j] = alpha * s + beta * C[i * n + j];
        }
    float *dA, *dB, *dC;
    const size_t bytes = sizeof(float) * n * n;
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&dA), bytes));
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&dB), bytes));
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&dC), bytes));
    HIP_OK(hipMemcpy(dA, A.data(), bytes, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(dB, B.data(), bytes, hipMemcpyHostToDevice));
    std::vector<float> got(n * n);
    for (int kernel = 1; kernel <= 5; ++kernel) {
        HIP_OK(hipMemcpy(dC, C.data(), bytes, hipMemcpyHostToDevice));
        run_my_kernel(kernel, n, n, n, alpha, dA, dB, beta, dC);
        HIP_OK(hipDeviceSynchronize());
        HIP_OK(hipGetLastError());
        HIP_OK(hipMemcpy(got.data(), dC, bytes, hipMemcpyDeviceToHost));
        for (int i = 0; i < n * n; ++i)
            if (!(std::fabs(got[i] - want[i]) <= 0.01)) {
                fprintf(stderr, "sgemm kernel %d: element %d is %f, expected %f\n", kernel, i, got[i], want[i]);
                return 1;
            }
        printf("sgemm kernel %d n=%d ok\n", kernel, n);
    }
    bool threw = false;
    try {
        run_my_kernel(9, n, n, n, alpha, dA, dB, beta, dC);  // runner.cu:265 throws std::invalid_argument
    } catch (const std::invalid_argument&) {
        threw = true;
    }
    HIP_OK(hipFree(dA));
    HIP_OK(hipFree(dB));
    HIP_OK(hipFree(dC));
    if (!threw) { fprintf(stderr, "sgemm: unknown kernel number did not throw\n"); return 1; }
    return 0;
}

// The workspace form on a skinny product (K cut across workgroups): against a host product, relative to the sums'
// size, and twice with the same bits.
static int check_sgemm_with_workspace(int M, int N, int K) {
    std::vector<float> A(static_cast<size_t>(M) * K), B(static_cast<size_t>(K) * N), C(static_cast<size_t>(M) * N);
    uint32_t seed = 5;
    for (auto* m : {&A, &B, &C})
        for (auto& v : *m) v = static_cast<float>(lcg(seed) % 5u) - 2.0f + 0.01f * static_cast<float>(lcg(seed) % 5u);
    const float alpha = 0.5f, beta = 3.0f;
    if (prism_sgemm_workspace_bytes(M, N, K) == 0) { fprintf(stderr, "sgemm: %dx%dx%d would not be cut\n", M, N, K); return 1; }
    float *dA, *dB, *dC;
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&dA), sizeof(float) * A.size()));
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&dB), sizeof(float) * B.size()));
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&dC), sizeof(float) * C.size()));
    HIP_OK(hipMemcpy(dA, A.data(), sizeof(float) * A.size(), hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(dB, B.data(), sizeof(float) * B.size(), hipMemcpyHostToDevice));
    std::vector<float> got(C.size()), again(C.size());
    for (auto* out : {&got, &again}) {
        HIP_OK(hipMemcpy(dC, C.data(), sizeof(float) * C.size(), hipMemcpyHostToDevice));
        run_my_sgemm_5_with_workspace(M, N, K, alpha, dA, dB, beta, dC);
        HIP_OK(hipDeviceSynchronize());
        HIP_OK(hipGetLastError());
        HIP_OK(hipMemcpy(out->data(), dC, sizeof(float) * C.size(), hipMemcpyDeviceToHost));
    }
    for (int i = 0; i < M; ++i)
        for (int j = 0; j < N; ++j) {
            double s = 0, mag = 0;
            for (int k = 0; k < K; ++k) {
                const double p = static_cast<double>(A[static_cast<size_t>(i) * K + k]) * B[static_cast<size_t>(k) * N + j];
                s += p;
                mag += std::fabs(p);
            }
            const double want = alpha * s + beta * C[static_cast<size_t>(i) * N + j];
            const float g = got[static_cast<size_t>(i) * N + j];
            if (!(std::fabs(g - want) <= 1e-5 * mag + 1e-4) || g != again[static_cast<size_t>(i) * N + j]) {
                fprintf(stderr, "sgemm with workspace: element (%d,%d) is %f / %f, expected %f\n", i, j, g,
                        again[static_cast<size_t>(i) * N + j], want);
                return 1;
            }
        }
    HIP_OK(hipFree(dA));
    HIP_OK(hipFree(dB));
    HIP_OK(hipFree(dC));
    printf("sgemm with workspace %dx%dx%d ok\n", M, N, K);
    return 0;
}

// evals/h100_bench/main.cu:123-141 in outline: bf16 C, column-major, |d| <= 0.1 (main.cu:48).
static int check_h100(int M, int N, int K) {
    std::vector<uint16_t> A(static_cast<size_t>(M) * K), B(static_cast<size_t>(N) * K);
    uint32_t seed = 11;
    for (auto* m : {&A, &B})
        for (auto& v : *m) v = to_bf16((static_cast<float>(lcg(seed) >> 8) / 8388608.0f - 1.0f));  // uniform in [-1, 1)
    uint16_t *dA, *dB, *dC;
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&dA), A.size() * 2));
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&dB), B.size() * 2));
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&dC), static_cast<size_t>(M) * N * 2));
    HIP_OK(hipMemcpy(dA, A.data(), A.size() * 2, hipMemcpyHostToDevice));
    HIP_OK(hipMemcpy(dB, B.data(), B.size() * 2, hipMemcpyHostToDevice));
    prism_h100::runmyh100(M, N, K, dA, dB, dC, nullptr);
    HIP_OK(hipDeviceSynchronize());
    HIP_OK(hipGetLastError());
    std::vector<uint16_t> C(static_cast<size_t>(M) * N);
    HIP_OK(hipMemcpy(C.data(), dC, C.size() * 2, hipMemcpyDeviceToHost));
    HIP_OK(hipFree(dA));
    HIP_OK(hipFree(dB));
    HIP_OK(hipFree(dC));
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            double s = 0;
            for (int k = 0; k < K; ++k)
                s += static_cast<double>(from_bf16(A[static_cast<size_t>(m) * K + k])) * from_bf16(B[static_cast<size_t>(n) * K + k]);
            const float got = from_bf16(C[static_cast<size_t>(n) * M + m]);  // column-major M x N
            if (!(std::fabs(got - s) <= 0.1)) {
                fprintf(stderr, "h100: C(%d,%d) is %f, expected %f\n", m, n, got, s);
                return 1;
            }
        }
    printf("h100 %dx%dx%d ok\n", M, N, K);
    return 0;
}

int main() {
    for (size_t n : {size_t{16384}, size_t{32768}, size_t{1} << 20, (size_t{1} << 20) + 17, size_t{1} << 24})
        if (check_scan(n)) return 1;
    if (check_sgemm(256)) return 1;
    if (check_sgemm_with_workspace(64, 256, 16384)) return 1;
    if (check_h100(256, 512, 192)) return 1;
    printf("OK\n");
    return 0;
}
