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
__global__ void handed_over_gemm(const __bf16* P, const __bf16* Q, float* D, int N, int K, int tiles_n) {
    extern __shared__ __align__(128) char __smem[];
    int __block_id_0 = blockIdx.x;
    int __thread_id_0 = __block_id_0 * blockDim.x + threadIdx.x;
    const int tile_r = (__block_id_0 / tiles_n);
    const int tile_c = (__block_id_0 % tiles_n);
    {
        const __bf16* P_rows = P + (((tile_r * 64) * K));
        {
            const __bf16* Q_rows = Q + (((tile_c * 64) * K));
            {
                float* D_tile = D + ((((tile_r * 64) * N) + (tile_c * 64)));
                {
                    int __block_id_1 = __block_id_0 % 1;
                    int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
                    __shared__ __bf16 p_first[2048];
                    __shared__ unsigned int __full_p_first, __empty_p_first;
                    int __round_p_first = 0;
                    bool __pending_p_first = false;  // filled by this wavefront and not announced yet
                    if (threadIdx.x == 0) { __full_p_first = 0; __empty_p_first = 0; }
                    __syncthreads();
                    __shared__ __bf16 q_first[2048];
                    __shared__ unsigned int __full_q_first, __empty_q_first;
                    int __round_q_first = 0;
                    bool __pending_q_first = false;  // filled by this wavefront and not announced yet
                    if (threadIdx.x == 0) { __full_q_first = 0; __empty_q_first = 0; }
                    __syncthreads();
                    __shared__ __bf16 p_second[2048];
                    __shared__ unsigned int __full_p_second, __empty_p_second;
                    int __round_p_second = 0;
                    bool __pending_p_second = false;  // filled by this wavefront and not announced yet
                    if (threadIdx.x == 0) { __full_p_second = 0; __empty_p_second = 0; }
                    __syncthreads();
                    __shared__ __bf16 q_second[2048];
                    __shared__ unsigned int __full_q_second, __empty_q_second;
                    int __round_q_second = 0;
                    bool __pending_q_second = false;  // filled by this wavefront and not announced yet
                    if (threadIdx.x == 0) { __full_q_second = 0; __empty_q_second = 0; }
                    __syncthreads();
                    float acc[16] = {0};
                    for (int k0 = 0; k0 < K; k0 += 64) {
                        {
                            __bf16* p_first_fill = p_first + (0);
                            {
                                __bf16* q_first_fill = q_first + (0);
                                {
                                    __bf16* p_second_fill = p_second + (0);
                                    {
                                        __bf16* q_second_fill = q_second + (0);
                                        {
                                            int __block_id_2 = __block_id_1;
                                            int __thread_id_2 = __thread_id_1;
                                            if (__thread_id_2 >= 0 && __thread_id_2 < 64) {
                                                {
                                                    int __block_id_3 = __block_id_2;
                                                    int __thread_id_3 = __thread_id_2 % 64;
                                                    int lane = __thread_id_3;
                                                    int row = (lane / 4);
                                                    int k8 = (8 * (lane % 4));
                                                    {
                                                        int __spin = 0;
                                                        const unsigned int __need = static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__round_p_first * 4)));
                                                        if (static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__prism_lds_peek(&__empty_p_first)))) < __need) {
                                                            if (__pending_p_first) {
                                                                __builtin_amdgcn_s_waitcnt(0);
                                                                if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_p_first);
                                                                __pending_p_first = false;
                                                            }
                                                            if (__pending_p_second) {
                                                                __builtin_amdgcn_s_waitcnt(0);
                                                                if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_p_second);
                                                                __pending_p_second = false;
                                                            }
                                                            if (__pending_q_first) {
                                                                __builtin_amdgcn_s_waitcnt(0);
                                                                if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_q_first);
                                                                __pending_q_first = false;
                                                            }
                                                            if (__pending_q_second) {
                                                                __builtin_amdgcn_s_waitcnt(0);
                                                                if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_q_second);
                                                                __pending_q_second = false;
                                                            }
                                                        }
                                                        #pragma nounroll
                                                        for (; __spin < 65536 && static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__prism_lds_peek(&__empty_p_first)))) < __need; ++__spin) __builtin_amdgcn_s_sleep(1);
                                                        if (__spin == 65536 && (threadIdx.x & 63) == 0) __hip_atomic_store(&__prism_handover_report, 1u | (static_cast<unsigned int>(__round_p_first) << 8), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                                                    }
                                                    {
                                                        int __spin = 0;
                                                        const unsigned int __need = static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__round_q_first * 4)));
                                                        if (static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__prism_lds_peek(&__empty_q_first)))) < __need) {
                                                            if (__pending_p_first) {
                                                                __builtin_amdgcn_s_waitcnt(0);
                                                                if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_p_first);
                                                                __pending_p_first = false;
                                                            }
                                                            if (__pending_p_second) {
                                                                __builtin_amdgcn_s_waitcnt(0);
                                                                if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_p_second);
                                                                __pending_p_second = false;
                                                            }
                                                            if (__pending_q_first) {
                                                                __builtin_amdgcn_s_waitcnt(0);
                                                                if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_q_first);
                                                                __pending_q_first = false;
                                                            }
                                                            if (__pending_q_second) {
                                                                __builtin_amdgcn_s_waitcnt(0);
                                                                if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_q_second);
                                                                __pending_q_second = false;
                                                            }
                                                        }
                                                        #pragma nounroll
                                                        for (; __spin < 65536 && static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__prism_lds_peek(&__empty_q_first)))) < __need; ++__spin) __builtin_amdgcn_s_sleep(1);
                                                        if (__spin == 65536 && (threadIdx.x & 63) == 0) __hip_atomic_store(&__prism_handover_report, 5u | (static_cast<unsigned int>(__round_q_first) << 8), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                                                    }
                                                    for (int part = 0; part < 4; part++) {
                                                        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(&P_rows[(((((16 * part) + row) * K) + k0) + k8)]), (__attribute__((address_space(3))) void*)(&p_first_fill[(512 * part)]), 16, 0, 0);
                                                        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(&Q_rows[(((((16 * part) + row) * K) + k0) + k8)]), (__attribute__((address_space(3))) void*)(&q_first_fill[(512 * part)]), 16, 0, 0);
                                                    }
                                                    __round_p_first += 1;
                                                    __round_q_first += 1;
                                                    if (__pending_p_second) {
                                                        __builtin_amdgcn_s_waitcnt(3960);  // vmcnt(8)
                                                        if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_p_second);
                                                        __pending_p_second = false;
                                                    }
                                                    if (__pending_q_second) {
                                                        __builtin_amdgcn_s_waitcnt(3960);  // vmcnt(8)
                                                        if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_q_second);
                                                        __pending_q_second = false;
                                                    }
                                                    __pending_p_first = true;
                                                    __pending_q_first = true;
                                                    {
                                                        int __spin = 0;
                                                        const unsigned int __need = static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__round_p_second * 4)));
                                                        if (static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__prism_lds_peek(&__empty_p_second)))) < __need) {
                                                            if (__pending_p_first) {
                                                                __builtin_amdgcn_s_waitcnt(0);
                                                                if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_p_first);
                                                                __pending_p_first = false;
                                                            }
                                                            if (__pending_p_second) {
                                                                __builtin_amdgcn_s_waitcnt(0);
                                                                if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_p_second);
                                                                __pending_p_second = false;
                                                            }
                                                            if (__pending_q_first) {
                                                                __builtin_amdgcn_s_waitcnt(0);
                                                                if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_q_first);
                                                                __pending_q_first = false;
                                                            }
                                                            if (__pending_q_second) {
                                                                __builtin_amdgcn_s_waitcnt(0);
                                                                if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_q_second);
                                                                __pending_q_second = false;
                                                            }
                                                        }
                                                        #pragma nounroll
                                                        for (; __spin < 65536 && static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__prism_lds_peek(&__empty_p_second)))) < __need; ++__spin) __builtin_amdgcn_s_sleep(1);
                                                        if (__spin == 65536 && (threadIdx.x & 63) == 0) __hip_atomic_store(&__prism_handover_report, 3u | (static_cast<unsigned int>(__round_p_second) << 8), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                                                    }
                                                    {
                                                        int __spin = 0;
                                                        const unsigned int __need = static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__round_q_second * 4)));
                                                        if (static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__prism_lds_peek(&__empty_q_second)))) < __need) {
                                                            if (__pending_p_first) {
                                                                __builtin_amdgcn_s_waitcnt(0);
                                                                if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_p_first);
                                                                __pending_p_first = false;
                                                            }
                                                            if (__pending_p_second) {
                                                                __builtin_amdgcn_s_waitcnt(0);
                                                                if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_p_second);
                                                                __pending_p_second = false;
                                                            }
                                                            if (__pending_q_first) {
                                                                __builtin_amdgcn_s_waitcnt(0);
                                                                if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_q_first);
                                                                __pending_q_first = false;
                                                            }
                                                            if (__pending_q_second) {
                                                                __builtin_amdgcn_s_waitcnt(0);
                                                                if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_q_second);
                                                                __pending_q_second = false;
                                                            }
                                                        }
                                                        #pragma nounroll
                                                        for (; __spin < 65536 && static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__prism_lds_peek(&__empty_q_second)))) < __need; ++__spin) __builtin_amdgcn_s_sleep(1);
                                                        if (__spin == 65536 && (threadIdx.x & 63) == 0) __hip_atomic_store(&__prism_handover_report, 7u | (static_cast<unsigned int>(__round_q_second) << 8), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                                                    }
                                                    for (int part = 0; part < 4; part++) {
                                                        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(&P_rows[((((((16 * part) + row) * K) + k0) + 32) + k8)]), (__attribute__((address_space(3))) void*)(&p_second_fill[(512 * part)]), 16, 0, 0);
                                                        __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(&Q_rows[((((((16 * part) + row) * K) + k0) + 32) + k8)]), (__attribute__((address_space(3))) void*)(&q_second_fill[(512 * part)]), 16, 0, 0);
                                                    }
                                                    __round_p_second += 1;
                                                    __round_q_second += 1;
                                                    if (__pending_p_first) {
                                                        __builtin_amdgcn_s_waitcnt(3960);  // vmcnt(8)
                                                        if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_p_first);
                                                        __pending_p_first = false;
                                                    }
                                                    if (__pending_q_first) {
                                                        __builtin_amdgcn_s_waitcnt(3960);  // vmcnt(8)
                                                        if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_q_first);
                                                        __pending_q_first = false;
                                                    }
                                                    __pending_p_second = true;
                                                    __pending_q_second = true;
                                                }
                                            }
                                        }
                                        {
                                            int __block_id_2 = __block_id_1;
                                            int __thread_id_2 = __thread_id_1 - 64;
                                            if (__thread_id_2 >= 0 && __thread_id_2 < 256) {
                                                int wave = (__thread_id_2 / 64);
                                                {
                                                    int __block_id_3 = __block_id_2;
                                                    int __thread_id_3 = __thread_id_2 % 64;
                                                    int lane = __thread_id_3;
                                                    int r = (lane % 16);
                                                    int k8 = (8 * (lane / 16));
                                                    {
                                                        int __spin = 0;
                                                        const unsigned int __need = static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>((__round_p_first + 1) * 1)));
                                                        #pragma nounroll
                                                        for (; __spin < 65536 && static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__hip_atomic_load(&__full_p_first, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP)))) < __need; ++__spin) __builtin_amdgcn_s_sleep(1);
                                                        if (__spin == 65536 && (threadIdx.x & 63) == 0) __hip_atomic_store(&__prism_handover_report, 2u | (static_cast<unsigned int>(__round_p_first) << 8), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                                                    }
                                                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
                                                    float4 a = reinterpret_cast<float4 *>(&p_first[((((16 * wave) + r) * 32) + k8)])[0];
                                                    __builtin_amdgcn_s_waitcnt(0);
                                                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
                                                    if ((threadIdx.x & 63) == 0) __hip_atomic_fetch_add(&__empty_p_first, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                                                    __round_p_first += 1;
                                                    {
                                                        int __spin = 0;
                                                        const unsigned int __need = static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>((__round_q_first + 1) * 1)));
                                                        #pragma nounroll
                                                        for (; __spin < 65536 && static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__hip_atomic_load(&__full_q_first, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP)))) < __need; ++__spin) __builtin_amdgcn_s_sleep(1);
                                                        if (__spin == 65536 && (threadIdx.x & 63) == 0) __hip_atomic_store(&__prism_handover_report, 6u | (static_cast<unsigned int>(__round_q_first) << 8), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                                                    }
                                                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
                                                    for (int n = 0; n < 4; n++) {
                                                        float4 b = reinterpret_cast<float4 *>(&q_first[((((16 * n) + r) * 32) + k8)])[0];
                                                        {
                                                            typedef float __acc_t __attribute__((ext_vector_type(4)));
                                                            __acc_t __acc = {acc[(4 * n)], acc[((4 * n) + 1)], acc[((4 * n) + 2)], acc[((4 * n) + 3)]};
                                                            typedef __bf16 __packet_t __attribute__((ext_vector_type(8)));
                                                            __acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(__packet_t, a), __builtin_bit_cast(__packet_t, b), __acc, 0, 0, 0);
                                                            acc[(4 * n)] = __acc[0];
                                                            acc[((4 * n) + 1)] = __acc[1];
                                                            acc[((4 * n) + 2)] = __acc[2];
                                                            acc[((4 * n) + 3)] = __acc[3];
                                                        }
                                                    }
                                                    __builtin_amdgcn_s_waitcnt(0);
                                                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
                                                    if ((threadIdx.x & 63) == 0) __hip_atomic_fetch_add(&__empty_q_first, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                                                    __round_q_first += 1;
                                                    {
                                                        int __spin = 0;
                                                        const unsigned int __need = static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>((__round_p_second + 1) * 1)));
                                                        #pragma nounroll
                                                        for (; __spin < 65536 && static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__hip_atomic_load(&__full_p_second, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP)))) < __need; ++__spin) __builtin_amdgcn_s_sleep(1);
                                                        if (__spin == 65536 && (threadIdx.x & 63) == 0) __hip_atomic_store(&__prism_handover_report, 4u | (static_cast<unsigned int>(__round_p_second) << 8), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                                                    }
                                                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
                                                    float4 a2 = reinterpret_cast<float4 *>(&p_second[((((16 * wave) + r) * 32) + k8)])[0];
                                                    __builtin_amdgcn_s_waitcnt(0);
                                                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
                                                    if ((threadIdx.x & 63) == 0) __hip_atomic_fetch_add(&__empty_p_second, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                                                    __round_p_second += 1;
                                                    {
                                                        int __spin = 0;
                                                        const unsigned int __need = static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>((__round_q_second + 1) * 1)));
                                                        #pragma nounroll
                                                        for (; __spin < 65536 && static_cast<unsigned int>(__builtin_amdgcn_readfirstlane(static_cast<int>(__hip_atomic_load(&__full_q_second, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP)))) < __need; ++__spin) __builtin_amdgcn_s_sleep(1);
                                                        if (__spin == 65536 && (threadIdx.x & 63) == 0) __hip_atomic_store(&__prism_handover_report, 8u | (static_cast<unsigned int>(__round_q_second) << 8), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                                                    }
                                                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
                                                    for (int n = 0; n < 4; n++) {
                                                        float4 b2 = reinterpret_cast<float4 *>(&q_second[((((16 * n) + r) * 32) + k8)])[0];
                                                        {
                                                            typedef float __acc_t __attribute__((ext_vector_type(4)));
                                                            __acc_t __acc = {acc[(4 * n)], acc[((4 * n) + 1)], acc[((4 * n) + 2)], acc[((4 * n) + 3)]};
                                                            typedef __bf16 __packet_t __attribute__((ext_vector_type(8)));
                                                            __acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(__packet_t, a2), __builtin_bit_cast(__packet_t, b2), __acc, 0, 0, 0);
                                                            acc[(4 * n)] = __acc[0];
                                                            acc[((4 * n) + 1)] = __acc[1];
                                                            acc[((4 * n) + 2)] = __acc[2];
                                                            acc[((4 * n) + 3)] = __acc[3];
                                                        }
                                                    }
                                                    __builtin_amdgcn_s_waitcnt(0);
                                                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
                                                    if ((threadIdx.x & 63) == 0) __hip_atomic_fetch_add(&__empty_q_second, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
                                                    __round_q_second += 1;
                                                }
                                            }
                                        }
                                    }
                                }
                            }
                        }
                    }
                    if (__pending_p_first) {
                        __builtin_amdgcn_s_waitcnt(0);
                        if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_p_first);
                        __pending_p_first = false;
                    }
                    if (__pending_p_second) {
                        __builtin_amdgcn_s_waitcnt(0);
                        if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_p_second);
                        __pending_p_second = false;
                    }
                    if (__pending_q_first) {
                        __builtin_amdgcn_s_waitcnt(0);
                        if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_q_first);
                        __pending_q_first = false;
                    }
                    if (__pending_q_second) {
                        __builtin_amdgcn_s_waitcnt(0);
                        if ((threadIdx.x & 63) == 0) __prism_lds_count(&__full_q_second);
                        __pending_q_second = false;
                    }
                    {
                        float* D_mine = D_tile + (0);
                        {
                            int __block_id_2 = __block_id_1;
                            int __thread_id_2 = __thread_id_1;
                            if (__thread_id_2 >= 0 && __thread_id_2 < 64) {
                            }
                        }
                        {
                            int __block_id_2 = __block_id_1;
                            int __thread_id_2 = __thread_id_1 - 64;
                            if (__thread_id_2 >= 0 && __thread_id_2 < 256) {
                                int wave = (__thread_id_2 / 64);
                                {
                                    int __block_id_3 = __block_id_2;
                                    int __thread_id_3 = __thread_id_2 % 64;
                                    int lane = __thread_id_3;
                                    {
                                        int __block_id_4 = __block_id_3;
                                        int __thread_id_4 = __thread_id_3 % 1;
                                        for (int n = 0; n < 4; n++) {
                                            for (int v = 0; v < 4; v++) {
                                                D_mine[((((((16 * wave) + (4 * (lane / 16))) + v) * N) + (16 * n)) + (lane % 16))] = acc[((4 * n) + v)];
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
