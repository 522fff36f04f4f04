#include <hip/hip_runtime.h>
#include <cstddef>
#include <cstdint>

__device__ void fill_slot_f32(int __block_id, int __thread_id, char* __smem, float* slot, const float* A_from, const float* B_from, int N, int K, int k_at) {
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
                int arow = ((8 * ((4 * part) + w)) + (lane / 8));
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(&A_from[(((arow * K) + k_at) + (4 * ((lane % 8) ^ ((arow / 2) % 8))))]), (__attribute__((address_space(3))) void*)(&slot[(256 * ((4 * part) + w))]), 16, 0, 0);
            }
            for (int part = 0; part < 8; part++) {
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(&B_from[((((k_at + (4 * part)) + w) * N) + (4 * lane))]), (__attribute__((address_space(3))) void*)(&slot[(4096 + (256 * ((4 * part) + w)))]), 16, 0, 0);
            }
        }
    }
    return;
}

__device__ void multiply_slot_f32(int __block_id, int __thread_id, char* __smem, float* acc, const float* slot) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0;
        int __thread_id_1 = __thread_id_0 % 512;
        int wave = (__thread_id_1 / 64);
        int row0 = (64 * (wave / 4));
        int col0 = (64 * (wave % 4));
        {
            int __block_id_2 = __block_id_1;
            int __thread_id_2 = __thread_id_1 % 64;
            int lane = __thread_id_2;
            int l32 = (lane % 32);
            float a[2];
            float b[2];
            for (int kk = 0; kk < 32; kk += 2) {
                int k = (kk + (lane / 32));
                for (int i = 0; i < 2; i++) {
                    a[i] = slot[(((((row0 + (32 * i)) + l32) * 32) + (4 * ((k / 4) ^ ((l32 / 2) % 8)))) + (k % 4))];
                }
                for (int j = 0; j < 2; j++) {
                    b[j] = slot[((((4096 + (k * 256)) + col0) + (32 * j)) + l32)];
                }
                for (int i = 0; i < 2; i++) {
                    for (int j = 0; j < 2; j++) {
                        {
                            typedef float __acc_t __attribute__((ext_vector_type(16)));
                            __acc_t __acc = {acc[((((2 * i) + j) * 16) + 0)], acc[((((2 * i) + j) * 16) + 1)], acc[((((2 * i) + j) * 16) + 2)], acc[((((2 * i) + j) * 16) + 3)], acc[((((2 * i) + j) * 16) + 4)], acc[((((2 * i) + j) * 16) + 5)], acc[((((2 * i) + j) * 16) + 6)], acc[((((2 * i) + j) * 16) + 7)], acc[((((2 * i) + j) * 16) + 8)], acc[((((2 * i) + j) * 16) + 9)], acc[((((2 * i) + j) * 16) + 10)], acc[((((2 * i) + j) * 16) + 11)], acc[((((2 * i) + j) * 16) + 12)], acc[((((2 * i) + j) * 16) + 13)], acc[((((2 * i) + j) * 16) + 14)], acc[((((2 * i) + j) * 16) + 15)]};
                            __acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], __acc, 0, 0, 0);
                            acc[((((2 * i) + j) * 16) + 0)] = __acc[0];
                            acc[((((2 * i) + j) * 16) + 1)] = __acc[1];
                            acc[((((2 * i) + j) * 16) + 2)] = __acc[2];
                            acc[((((2 * i) + j) * 16) + 3)] = __acc[3];
                            acc[((((2 * i) + j) * 16) + 4)] = __acc[4];
                            acc[((((2 * i) + j) * 16) + 5)] = __acc[5];
                            acc[((((2 * i) + j) * 16) + 6)] = __acc[6];
                            acc[((((2 * i) + j) * 16) + 7)] = __acc[7];
                            acc[((((2 * i) + j) * 16) + 8)] = __acc[8];
                            acc[((((2 * i) + j) * 16) + 9)] = __acc[9];
                            acc[((((2 * i) + j) * 16) + 10)] = __acc[10];
                            acc[((((2 * i) + j) * 16) + 11)] = __acc[11];
                            acc[((((2 * i) + j) * 16) + 12)] = __acc[12];
                            acc[((((2 * i) + j) * 16) + 13)] = __acc[13];
                            acc[((((2 * i) + j) * 16) + 14)] = __acc[14];
                            acc[((((2 * i) + j) * 16) + 15)] = __acc[15];
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
__global__ __launch_bounds__(768) void handed_over_sgemm(int M, int N, int K, float alpha, const float* A, const float* B, float beta, float* C, int tiles_n) {
    extern __shared__ __align__(128) char __smem[];
    int __block_id_0 = blockIdx.x;
    int __thread_id_0 = __block_id_0 * blockDim.x + threadIdx.x;
    const int per_xcd = (((M / 128) * tiles_n) / 8);
    const int t = (((__block_id_0 % 8) * per_xcd) + (__block_id_0 / 8));
    const int tile_r = ((8 * (t / (8 * tiles_n))) + (t % 8));
    const int tile_c = ((t % (8 * tiles_n)) / 8);
    {
        const float* A_rows = A + (((tile_r * 128) * K));
        {
            const float* B_cols = B + ((tile_c * 256));
            {
                float* C_tile = C + ((((tile_r * 128) * N) + (tile_c * 256)));
                {
                    int __block_id_1 = __block_id_0 % 1;
                    int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
                    __shared__ float first[12288];
                    __shared__ unsigned int __full_first, __empty_first;
                    int __round_first = 0;
                    bool __pending_first = false;  // filled by this wavefront and not announced yet
                    if (threadIdx.x == 0) { __full_first = 0; __empty_first = 0; }
                    __syncthreads();
                    __shared__ float second[12288];
                    __shared__ unsigned int __full_second, __empty_second;
                    int __round_second = 0;
                    bool __pending_second = false;  // filled by this wavefront and not announced yet
                    if (threadIdx.x == 0) { __full_second = 0; __empty_second = 0; }
                    __syncthreads();
                    float acc[64] = {0};
                    for (int k0 = 0; k0 < K; k0 += 64) {
                        {
                            float* first_fill = first + (0);
                            {
                                float* second_fill = second + (0);
                                {
                                    int __block_id_2 = __block_id_1;
                                    int __thread_id_2 = __thread_id_1;
                                    if (__thread_id_2 >= 0 && __thread_id_2 < 256) {
                                        {
                                            int __spin = 0;
                                            const unsigned int __need = static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__round_first * 8)));
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
                                            }
                                            #pragma nounroll
                                            for (; __spin < 65536 && static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__prism_lds_peek(&__empty_first)))) < __need; ++__spin) __builtin_amdgcn_s_sleep(1);
                                            if (__spin == 65536 && (threadIdx.x & 63) == 0) __hip_atomic_store(&__prism_handover_report, 1u | (static_cast<unsigned int>(__round_first) << 8), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                                        }
                                        fill_slot_f32(__block_id_2, __thread_id_2, __smem, first_fill, A_rows, B_cols, N, K, k0);
                                        __round_first += 1;
                                        if (__pending_second) {
                                            __builtin_amdgcn_s_waitcnt(3964);  // vmcnt(12)
                                            if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_second);
                                            __pending_second = false;
                                        }
                                        __pending_first = true;
                                        {
                                            int __spin = 0;
                                            const unsigned int __need = static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__round_second * 8)));
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
                                            }
                                            #pragma nounroll
                                            for (; __spin < 65536 && static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__prism_lds_peek(&__empty_second)))) < __need; ++__spin) __builtin_amdgcn_s_sleep(1);
                                            if (__spin == 65536 && (threadIdx.x & 63) == 0) __hip_atomic_store(&__prism_handover_report, 3u | (static_cast<unsigned int>(__round_second) << 8), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                                        }
                                        fill_slot_f32(__block_id_2, __thread_id_2, __smem, second_fill, A_rows, B_cols, N, K, (k0 + 32));
                                        __round_second += 1;
                                        if (__pending_first) {
                                            __builtin_amdgcn_s_waitcnt(3964);  // vmcnt(12)
                                            if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_first);
                                            __pending_first = false;
                                        }
                                        __pending_second = true;
                                    }
                                }
                                {
                                    int __block_id_2 = __block_id_1;
                                    int __thread_id_2 = __thread_id_1 - 256;
                                    if (__thread_id_2 >= 0 && __thread_id_2 < 512) {
                                        {
                                            int __spin = 0;
                                            const unsigned int __need = static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>((__round_first + 1) * 4)));
                                            #pragma nounroll
                                            for (; __spin < 65536 && static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__hip_atomic_load(&__full_first, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP)))) < __need; ++__spin) __builtin_amdgcn_s_sleep(1);
                                            if (__spin == 65536 && (threadIdx.x & 63) == 0) __hip_atomic_store(&__prism_handover_report, 2u | (static_cast<unsigned int>(__round_first) << 8), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                                        }
                                        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
                                        multiply_slot_f32(__block_id_2, __thread_id_2, __smem, acc, first);
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
                                        multiply_slot_f32(__block_id_2, __thread_id_2, __smem, acc, second);
                                        __builtin_amdgcn_s_waitcnt(0);
                                        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
                                        if ((threadIdx.x & 63) == 0) __hip_atomic_fetch_add(&__empty_second, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                                        __round_second += 1;
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
                    {
                        float* C_mine = C_tile + (0);
                        {
                            int __block_id_2 = __block_id_1;
                            int __thread_id_2 = __thread_id_1;
                            if (__thread_id_2 >= 0 && __thread_id_2 < 256) {
                            }
                        }
                        {
                            int __block_id_2 = __block_id_1;
                            int __thread_id_2 = __thread_id_1 - 256;
                            if (__thread_id_2 >= 0 && __thread_id_2 < 512) {
                                int wave = (__thread_id_2 / 64);
                                {
                                    int __block_id_3 = __block_id_2;
                                    int __thread_id_3 = __thread_id_2 % 64;
                                    int lane = __thread_id_3;
                                    {
                                        int __block_id_4 = __block_id_3;
                                        int __thread_id_4 = __thread_id_3 % 1;
                                        for (int i = 0; i < 2; i++) {
                                            for (int j = 0; j < 2; j++) {
                                                for (int v = 0; v < 16; v++) {
                                                    int at = (((((((((64 * (wave / 4)) + (32 * i)) + (8 * (v / 4))) + (4 * (lane / 32))) + (v % 4)) * N) + (64 * (wave % 4))) + (32 * j)) + (lane % 32));
                                                    C_mine[at] = ((alpha * acc[((((2 * i) + j) * 16) + v)]) + (beta * C_mine[at]));
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

extern "C" int handed_over_sgemm_launch(int M, int N, int K, float alpha, const float* A, const float* B, float beta, float* C, int tiles_n, unsigned grid_blocks, void* stream) {
    if (grid_blocks == 0) return 0;
    handed_over_sgemm<<<dim3(grid_blocks), dim3(768), 0, static_cast<hipStream_t>(stream)>>>(M, N, K, alpha, A, B, beta, C, tiles_n);
    return static_cast<int>(hipGetLastError());
}

extern "C" int handed_over_sgemm_status(void* stream) {
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
