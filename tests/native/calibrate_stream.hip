// Streaming calibration kernels: what this GPU's memory system gives a kernel that only moves bytes,
// in the two access shapes the streaming kernels of libprism_amd.so use. bench.py times them next to
// add_m and the scan (the ceiling those are measured against besides the published 8 TB/s) and scales
// the FETCH_SIZE / WRITE_SIZE counters by what they read for a copy of known size. A measurement aid:
// built into its own small library (libcalibrate_stream.so, see tests/calibrate_stream.py), not part of
// the product library or its header.
//
//   int calibrate_stream(int kind, const void* in, void* out, size_t bytes, void* stream)
//       0 = launched; 1 = bad argument; otherwise the hipError_t of the launch. `bytes` is a multiple of
//       16, both buffers 16-byte aligned.
//
//   kind 0  copy, one 16 B packet per lane, 256-thread workgroups (add_m's shape): the workgroups sweep
//           memory in dispatch order as one compact front
//   kind 1  copy, 1024 threads x 16 packets per lane, a wave owns 16 KiB (the scan's big tile): every
//           workgroup loads its whole 256 KiB tile, then stores it
//   kind 2  read only, shape of kind 0 (4 bytes per workgroup are written so that the loads are kept)
//   kind 3  write only, shape of kind 0
#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

namespace {

constexpr int kWave = 64;

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void stream_store(u32x4* p, u32x4 v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\ts_nop 1" ::"v"(p), "v"(v) : "memory");
}

__global__ __launch_bounds__(256) void calibrate_copy_packet_kernel(const u32x4* __restrict__ in, u32x4* __restrict__ out,
                                                                    size_t n_vec) {
    const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i < n_vec) stream_store(&out[i], __builtin_nontemporal_load(&in[i]));
}

constexpr int kTileThreads = 1024, kTilePackets = 16;

__global__ __launch_bounds__(kTileThreads) void calibrate_copy_tile_kernel(const u32x4* __restrict__ in,
                                                                           u32x4* __restrict__ out, size_t n_vec) {
    const size_t base = static_cast<size_t>(blockIdx.x) * kTileThreads * kTilePackets +
                        (threadIdx.x / kWave) * kWave * kTilePackets + (threadIdx.x % kWave);
    u32x4 v[kTilePackets];
#pragma unroll
    for (int j = 0; j < kTilePackets; ++j)
        if (base + j * kWave < n_vec) v[j] = __builtin_nontemporal_load(&in[base + j * kWave]);
#pragma unroll
    for (int j = 0; j < kTilePackets; ++j)
        if (base + j * kWave < n_vec) stream_store(&out[base + j * kWave], v[j]);
}

__global__ __launch_bounds__(256) void calibrate_read_kernel(const u32x4* __restrict__ in, uint32_t* sink, size_t n_vec) {
    const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (i < n_vec) v = __builtin_nontemporal_load(&in[i]);
    // One lane in 2^32 data patterns writes: the loads cannot be dropped, the store traffic is nil.
    if ((v.x ^ v.y ^ v.z ^ v.w) == 0x9e3779b9u && threadIdx.x == 0) sink[blockIdx.x % 64] = v.x;
}

__global__ __launch_bounds__(256) void calibrate_write_kernel(u32x4* __restrict__ out, size_t n_vec) {
    const size_t i = static_cast<size_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i < n_vec) stream_store(&out[i], u32x4{static_cast<uint32_t>(i), 1u, 2u, 3u});
}

}  // namespace

extern "C" int calibrate_stream(int kind, const void* in, void* out, size_t bytes, void* stream) {
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (kind < 0 || kind > 3) return 1;
    if (bytes == 0) return 0;
    if ((kind != 3 && in == nullptr) || out == nullptr) return 1;
    if (bytes % 16 != 0 || (reinterpret_cast<uintptr_t>(in) & 15u) || (reinterpret_cast<uintptr_t>(out) & 15u)) return 1;
    if (kind == 2 && bytes < 256) return 1;  // the read-only kind writes into the first 256 bytes of `out`
    const size_t n_vec = bytes / 16;
    const size_t per_block = kind == 1 ? static_cast<size_t>(kTileThreads) * kTilePackets : 256;
    const size_t blocks = (n_vec + per_block - 1) / per_block;
    if (blocks > 0x7fffffffull) return 1;
    const dim3 grid(static_cast<unsigned>(blocks));
    const u32x4* src = static_cast<const u32x4*>(in);
    u32x4* dst = static_cast<u32x4*>(out);
    switch (kind) {
        case 0: calibrate_copy_packet_kernel<<<grid, dim3(256), 0, s>>>(src, dst, n_vec); break;
        case 1: calibrate_copy_tile_kernel<<<grid, dim3(kTileThreads), 0, s>>>(src, dst, n_vec); break;
        case 2: calibrate_read_kernel<<<grid, dim3(256), 0, s>>>(src, static_cast<uint32_t*>(out), n_vec); break;
        default: calibrate_write_kernel<<<grid, dim3(256), 0, s>>>(dst, n_vec); break;
    }
    return static_cast<int>(hipGetLastError());
}
