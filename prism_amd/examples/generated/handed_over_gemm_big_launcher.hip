#include <hip/hip_runtime.h>
#include <cstddef>
#include <cstdint>

__device__ void fill_slot(int __block_id, int __thread_id, char* __smem, __bf16* slot, const __bf16* P_from, const __bf16* Q_from, int K, int k_at) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0;
        int __thread_id_1 = __thread_id_0 % 256;
        int w = (__thread_id_1 / 64);
        {
            int __block_id_2 = __block_id_1;
            int __thread_id_2 = __thread_id_1 % 64;
            int lane = __thread_id_2;
            for (int part = 0; part < 4; part++) {
                int prow = ((8 * ((4 * part) + w)) + (lane / 8));
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(&P_from[(((prow * K) + k_at) + (8 * ((lane % 8) ^ ((prow / 2) % 8))))]), (__attribute__((address_space(3))) void*)(&slot[(512 * ((4 * part) + w))]), 16, 0, 0);
            }
            for (int part = 0; part < 8; part++) {
                int qrow = ((8 * ((4 * part) + w)) + (lane / 8));
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(&Q_from[(((qrow * K) + k_at) + (8 * ((lane % 8) ^ ((qrow / 2) % 8))))]), (__attribute__((address_space(3))) void*)(&slot[(8192 + (512 * ((4 * part) + w)))]), 16, 0, 0);
            }
        }
    }
    return;
}

__device__ void multiply_slot(int __block_id, int __thread_id, char* __smem, float* acc, const __bf16* slot) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0;
        int __thread_id_1 = __thread_id_0 % 256;
        int wave = (__thread_id_1 / 64);
        int row0 = (64 * (wave / 2));
        int col0 = (128 * (wave % 2));
        {
            int __block_id_2 = __block_id_1;
            int __thread_id_2 = __thread_id_1 % 64;
            int lane = __thread_id_2;
            int r = (lane % 16);
            float4 a[4];
            for (int kk = 0; kk < 2; kk++) {
                int k8 = (8 * (((4 * kk) + (lane / 16)) ^ ((r / 2) % 8)));
                for (int i = 0; i < 4; i++) {
                    a[i] = reinterpret_cast<const float4 *>(&slot[((((row0 + (16 * i)) + r) * 64) + k8)])[0];
                }
                for (int j = 0; j < 8; j++) {
                    float4 b = reinterpret_cast<const float4 *>(&slot[((8192 + (((col0 + (16 * j)) + r) * 64)) + k8)])[0];
                    for (int i = 0; i < 4; i++) {
                        {
                            typedef float __acc_t __attribute__((ext_vector_type(4)));
                            __acc_t __acc = {acc[(((8 * i) + j) * 4)], acc[((((8 * i) + j) * 4) + 1)], acc[((((8 * i) + j) * 4) + 2)], acc[((((8 * i) + j) * 4) + 3)]};
                            typedef __bf16 __packet_t __attribute__((ext_vector_type(8)));
                            __acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(__packet_t, a[i]), __builtin_bit_cast(__packet_t, b), __acc, 0, 0, 0);
                            acc[(((8 * i) + j) * 4)] = __acc[0];
                            acc[((((8 * i) + j) * 4) + 1)] = __acc[1];
                            acc[((((8 * i) + j) * 4) + 2)] = __acc[2];
                            acc[((((8 * i) + j) * 4) + 3)] = __acc[3];
                        }
                    }
                }
            }
        }
    }
    return;
}

#ifndef PRISM_HANDOVER_REPORT
#define PRISM_HANDOVER_REPORT
// written by a hand-over wait that ran out of polls: 1 + 2 * (array number) + (1 when waiting for a filled
// array) in the low byte, the round above it; the launcher's <name>_status call reads and clears it
__device__ unsigned int __prism_handover_report = 0;
#endif
#ifndef PRISM_LDS_WORD_HELPERS
#define PRISM_LDS_WORD_HELPERS
// one LDS word read / counted up without the compiler seeing an LDS access (the address is the low half of the
// generic one); the memory clobber keeps every memory operation on its side of the call
__device__ __forceinline__ unsigned int __prism_lds_peek(const unsigned int* word) {
    unsigned int value;
    asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(0)" : "=v"(value) : "v"((unsigned int)(unsigned long long)word) : "memory");
    return value;
}
__device__ __forceinline__ void __prism_lds_count(unsigned int* word) {
    asm volatile("ds_add_u32 %0, %1" :: "v"((unsigned int)(unsigned long long)word), "v"(1u) : "memory");
}
#endif
__global__ __launch_bounds__(512) void handed_over_gemm_big(const __bf16* P, const __bf16* Q, float* D, int N, int K, int tiles_m, int tiles_n) {
    extern __shared__ __align__(128) char __smem[];
    int __block_id_0 = blockIdx.x;
    int __thread_id_0 = __block_id_0 * blockDim.x + threadIdx.x;
    const int per_xcd = ((tiles_m * tiles_n) / 8);
    const int t = (((__block_id_0 % 8) * per_xcd) + (__block_id_0 / 8));
    const int tile_r = ((8 * (t / (8 * tiles_n))) + (t % 8));
    const int tile_c = ((t % (8 * tiles_n)) / 8);
    {
        const __bf16* P_rows = P + (((tile_r * 128) * K));
        {
            const __bf16* Q_rows = Q + (((tile_c * 256) * K));
            {
                float* D_tile = D + ((((tile_r * 128) * N) + (tile_c * 256)));
                {
                    int __block_id_1 = __block_id_0 % 1;
                    int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
                    __shared__ __bf16 first[24576];
                    __shared__ unsigned int __full_first, __empty_first;
                    int __round_first = 0;
                    bool __pending_first = false;  // filled by this wavefront and not announced yet
                    if (threadIdx.x == 0) { __full_first = 0; __empty_first = 0; }
                    __syncthreads();
                    __shared__ __bf16 second[24576];
                    __shared__ unsigned int __full_second, __empty_second;
                    int __round_second = 0;
                    bool __pending_second = false;  // filled by this wavefront and not announced yet
                    if (threadIdx.x == 0) { __full_second = 0; __empty_second = 0; }
                    __syncthreads();
                    __shared__ __bf16 third[24576];
                    __shared__ unsigned int __full_third, __empty_third;
                    int __round_third = 0;
                    bool __pending_third = false;  // filled by this wavefront and not announced yet
                    if (threadIdx.x == 0) { __full_third = 0; __empty_third = 0; }
                    __syncthreads();
                    float acc[128] = {0};
                    for (int k0 = 0; k0 < K; k0 += 192) {
                        const int k1 = ((k0 + 64) % K);
                        const int k2 = ((k0 + 128) % K);
                        {
                            __bf16* first_fill = first + (0);
                            {
                                __bf16* second_fill = second + (0);
                                {
                                    __bf16* third_fill = third + (0);
                                    {
                                        int __block_id_2 = __block_id_1;
                                        int __thread_id_2 = __thread_id_1;
                                        if (__thread_id_2 >= 0 && __thread_id_2 < 256) {
                                            {
                                                int __spin = 0;
                                                const unsigned int __need = static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__round_first * 4)));
                                                if (static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__prism_lds_peek(&__empty_first)))) < __need) {
                                                    if (__pending_first) {
                                                        __builtin_amdgcn_s_waitcnt(0);
                                                        if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_first);
                                                        __pending_first = false;
                                                    }
                                                    if (__pending_second) {
                                                        __builtin_amdgcn_s_waitcnt(0);
                                                        if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_second);
                                                        __pending_second = false;
                                                    }
                                                    if (__pending_third) {
                                                        __builtin_amdgcn_s_waitcnt(0);
                                                        if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_third);
                                                        __pending_third = false;
                                                    }
                                                }
                                                #pragma nounroll
                                                for (; __spin < 65536 && static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__prism_lds_peek(&__empty_first)))) < __need; ++__spin) __builtin_amdgcn_s_sleep(1);
                                                if (__spin == 65536 && (threadIdx.x & 63) == 0) __hip_atomic_store(&__prism_handover_report, 1u | (static_cast<unsigned int>(__round_first) << 8), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                                            }
                                            fill_slot(__block_id_2, __thread_id_2, __smem, first_fill, P_rows, Q_rows, K, k0);
                                            __round_first += 1;
                                            if (__pending_second) {
                                                __builtin_amdgcn_s_waitcnt(3964);  // vmcnt(12)
                                                if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_second);
                                                __pending_second = false;
                                            }
                                            if (__pending_third) {
                                                __builtin_amdgcn_s_waitcnt(3964);  // vmcnt(12)
                                                if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_third);
                                                __pending_third = false;
                                            }
                                            __pending_first = true;
                                            {
                                                int __spin = 0;
                                                const unsigned int __need = static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__round_second * 4)));
                                                if (static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__prism_lds_peek(&__empty_second)))) < __need) {
                                                    if (__pending_first) {
                                                        __builtin_amdgcn_s_waitcnt(0);
                                                        if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_first);
                                                        __pending_first = false;
                                                    }
                                                    if (__pending_second) {
                                                        __builtin_amdgcn_s_waitcnt(0);
                                                        if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_second);
                                                        __pending_second = false;
                                                    }
                                                    if (__pending_third) {
                                                        __builtin_amdgcn_s_waitcnt(0);
                                                        if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_third);
                                                        __pending_third = false;
                                                    }
                                                }
                                                #pragma nounroll
                                                for (; __spin < 65536 && static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__prism_lds_peek(&__empty_second)))) < __need; ++__spin) __builtin_amdgcn_s_sleep(1);
                                                if (__spin == 65536 && (threadIdx.x & 63) == 0) __hip_atomic_store(&__prism_handover_report, 3u | (static_cast<unsigned int>(__round_second) << 8), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                                            }
                                            fill_slot(__block_id_2, __thread_id_2, __smem, second_fill, P_rows, Q_rows, K, k1);
                                            __round_second += 1;
                                            if (__pending_first) {
                                                __builtin_amdgcn_s_waitcnt(3964);  // vmcnt(12)
                                                if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_first);
                                                __pending_first = false;
                                            }
                                            if (__pending_third) {
                                                __builtin_amdgcn_s_waitcnt(3964);  // vmcnt(12)
                                                if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_third);
                                                __pending_third = false;
                                            }
                                            __pending_second = true;
                                            {
                                                int __spin = 0;
                                                const unsigned int __need = static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__round_third * 4)));
                                                if (static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__prism_lds_peek(&__empty_third)))) < __need) {
                                                    if (__pending_first) {
                                                        __builtin_amdgcn_s_waitcnt(0);
                                                        if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_first);
                                                        __pending_first = false;
                                                    }
                                                    if (__pending_second) {
                                                        __builtin_amdgcn_s_waitcnt(0);
                                                        if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_second);
                                                        __pending_second = false;
                                                    }
                                                    if (__pending_third) {
                                                        __builtin_amdgcn_s_waitcnt(0);
                                                        if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_third);
                                                        __pending_third = false;
                                                    }
                                                }
                                                #pragma nounroll
                                                for (; __spin < 65536 && static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__prism_lds_peek(&__empty_third)))) < __need; ++__spin) __builtin_amdgcn_s_sleep(1);
                                                if (__spin == 65536 && (threadIdx.x & 63) == 0) __hip_atomic_store(&__prism_handover_report, 5u | (static_cast<unsigned int>(__round_third) << 8), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                                            }
                                            fill_slot(__block_id_2, __thread_id_2, __smem, third_fill, P_rows, Q_rows, K, k2);
                                            __round_third += 1;
                                            if (__pending_first) {
                                                __builtin_amdgcn_s_waitcnt(3964);  // vmcnt(12)
                                                if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_first);
                                                __pending_first = false;
                                            }
                                            if (__pending_second) {
                                                __builtin_amdgcn_s_waitcnt(3964);  // vmcnt(12)
                                                if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_second);
                                                __pending_second = false;
                                            }
                                            __pending_third = true;
                                        }
                                    }
                                    {
                                        int __block_id_2 = __block_id_1;
                                        int __thread_id_2 = __thread_id_1 - 256;
                                        if (__thread_id_2 >= 0 && __thread_id_2 < 256) {
                                            {
                                                int __spin = 0;
                                                const unsigned int __need = static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>((__round_first + 1) * 4)));
                                                #pragma nounroll
                                                for (; __spin < 65536 && static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__hip_atomic_load(&__full_first, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP)))) < __need; ++__spin) __builtin_amdgcn_s_sleep(1);
                                                if (__spin == 65536 && (threadIdx.x & 63) == 0) __hip_atomic_store(&__prism_handover_report, 2u | (static_cast<unsigned int>(__round_first) << 8), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                                            }
                                            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
                                            multiply_slot(__block_id_2, __thread_id_2, __smem, acc, first);
                                            __builtin_amdgcn_s_waitcnt(0);
                                            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
                                            if ((threadIdx.x & 63) == 0) __hip_atomic_fetch_add(&__empty_first, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                                            __round_first += 1;
                                            {
                                                int __spin = 0;
                                                const unsigned int __need = static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>((__round_second + 1) * 4)));
                                                #pragma nounroll
                                                for (; __spin < 65536 && static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__hip_atomic_load(&__full_second, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP)))) < __need; ++__spin) __builtin_amdgcn_s_sleep(1);
                                                if (__spin == 65536 && (threadIdx.x & 63) == 0) __hip_atomic_store(&__prism_handover_report, 4u | (static_cast<unsigned int>(__round_second) << 8), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                                            }
                                            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
                                            if (((k0 + 64) < K)) {
                                                multiply_slot(__block_id_2, __thread_id_2, __smem, acc, second);
                                            }
                                            __builtin_amdgcn_s_waitcnt(0);
                                            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
                                            if ((threadIdx.x & 63) == 0) __hip_atomic_fetch_add(&__empty_second, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                                            __round_second += 1;
                                            {
                                                int __spin = 0;
                                                const unsigned int __need = static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>((__round_third + 1) * 4)));
                                                #pragma nounroll
                                                for (; __spin < 65536 && static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__hip_atomic_load(&__full_third, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP)))) < __need; ++__spin) __builtin_amdgcn_s_sleep(1);
                                                if (__spin == 65536 && (threadIdx.x & 63) == 0) __hip_atomic_store(&__prism_handover_report, 6u | (static_cast<unsigned int>(__round_third) << 8), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                                            }
                                            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
                                            if (((k0 + 128) < K)) {
                                                multiply_slot(__block_id_2, __thread_id_2, __smem, acc, third);
                                            }
                                            __builtin_amdgcn_s_waitcnt(0);
                                            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
                                            if ((threadIdx.x & 63) == 0) __hip_atomic_fetch_add(&__empty_third, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                                            __round_third += 1;
                                        }
                                    }
                                }
                            }
                        }
                    }
                    if (__pending_first) {
                        __builtin_amdgcn_s_waitcnt(0);
                        if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_first);
                        __pending_first = false;
                    }
                    if (__pending_second) {
                        __builtin_amdgcn_s_waitcnt(0);
                        if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_second);
                        __pending_second = false;
                    }
                    if (__pending_third) {
                        __builtin_amdgcn_s_waitcnt(0);
                        if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_third);
                        __pending_third = false;
                    }
                    {
                        float* D_mine = D_tile + (0);
                        {
                            int __block_id_2 = __block_id_1;
                            int __thread_id_2 = __thread_id_1;
                            if (__thread_id_2 >= 0 && __thread_id_2 < 256) {
                            }
                        }
                        {
                            int __block_id_2 = __block_id_1;
                            int __thread_id_2 = __thread_id_1 - 256;
                            if (__thread_id_2 >= 0 && __thread_id_2 < 256) {
                                int wave = (__thread_id_2 / 64);
                                {
                                    int __block_id_3 = __block_id_2;
                                    int __thread_id_3 = __thread_id_2 % 64;
                                    int lane = __thread_id_3;
                                    {
                                        int __block_id_4 = __block_id_3;
                                        int __thread_id_4 = __thread_id_3 % 1;
                                        for (int i = 0; i < 4; i++) {
                                            for (int j = 0; j < 8; j++) {
                                                for (int v = 0; v < 4; v++) {
                                                    D_mine[((((((((64 * (wave / 2)) + (16 * i)) + (4 * (lane / 16))) + v) * N) + (128 * (wave % 2))) + (16 * j)) + (lane % 16))] = acc[((((8 * i) + j) * 4) + v)];
                                                }
                                            }
                                        }
                                    }
                                }
                            }
                        }
                    }
                }
            }
        }
    }
}

extern "C" int handed_over_gemm_big_launch(const __bf16* P, const __bf16* Q, float* D, int N, int K, int tiles_m, int tiles_n, unsigned grid_blocks, void* stream) {
    if (grid_blocks == 0) return 0;
    handed_over_gemm_big<<<dim3(grid_blocks), dim3(512), 0, static_cast<hipStream_t>(stream)>>>(P, Q, D, N, K, tiles_m, tiles_n);
    return static_cast<int>(hipGetLastError());
}

extern "C" int handed_over_gemm_big_status(void* stream) {
    hipError_t e = hipStreamSynchronize(static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return static_cast<int>(e);
    unsigned int word = 0;
    e = hipMemcpyFromSymbol(&word, HIP_SYMBOL(__prism_handover_report), sizeof(word));
    if (e != hipSuccess) return static_cast<int>(e);
    if (word == 0) return 0;
    const unsigned int zero = 0;
    e = hipMemcpyToSymbol(HIP_SYMBOL(__prism_handover_report), &zero, sizeof(zero));
    if (e != hipSuccess) return static_cast<int>(e);
    return static_cast<int>(0x40000000u | (word & 0x3fffffffu));
}
