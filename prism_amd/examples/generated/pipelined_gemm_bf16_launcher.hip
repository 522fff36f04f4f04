#include <hip/hip_runtime.h>
#include <cstddef>
#include <cstdint>

__device__ void fill_stage_bf16(int __block_id, int __thread_id, char* __smem, __bf16* stage, const __bf16* P_from, const __bf16* Q_from, int K, int k_at) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0;
        int __thread_id_1 = __thread_id_0 % 512;
        int w = (__thread_id_1 / 64);
        {
            int __block_id_2 = __block_id_1;
            int __thread_id_2 = __thread_id_1 % 64;
            int lane = __thread_id_2;
            for (int part = 0; part < 4; part++) {
                int prow = ((8 * ((8 * part) + w)) + (lane / 8));
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(&P_from[(((prow * K) + k_at) + (8 * ((lane % 8) ^ ((prow / 2) % 8))))]), (__attribute__((address_space(3))) void*)(&stage[(512 * ((8 * part) + w))]), 16, 0, 0);
            }
            for (int part = 0; part < 4; part++) {
                int qrow = ((8 * ((8 * part) + w)) + (lane / 8));
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(&Q_from[(((qrow * K) + k_at) + (8 * ((lane % 8) ^ ((qrow / 2) % 8))))]), (__attribute__((address_space(3))) void*)(&stage[(16384 + (512 * ((8 * part) + w)))]), 16, 0, 0);
            }
        }
    }
    return;
}

__device__ void multiply_stage_bf16(int __block_id, int __thread_id, char* __smem, float* acc, const __bf16* stage) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0;
        int __thread_id_1 = __thread_id_0 % 512;
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
                    a[i] = reinterpret_cast<const float4 *>(&stage[((((row0 + (16 * i)) + r) * 64) + k8)])[0];
                }
                for (int j = 0; j < 8; j++) {
                    float4 b = reinterpret_cast<const float4 *>(&stage[((16384 + (((col0 + (16 * j)) + r) * 64)) + k8)])[0];
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

__global__ __launch_bounds__(512) void pipelined_gemm_bf16(const __bf16* P, const __bf16* Q, float* D, int N, int K, int tiles_m, int tiles_n) {
    extern __shared__ __align__(128) char __smem[];
    int __block_id_0 = blockIdx.x;
    int __thread_id_0 = __block_id_0 * blockDim.x + threadIdx.x;
    const int per_xcd = ((tiles_m * tiles_n) / 8);
    const int t = (((__block_id_0 % 8) * per_xcd) + (__block_id_0 / 8));
    const int tile_r = ((8 * (t / (8 * tiles_n))) + (t % 8));
    const int tile_c = ((t % (8 * tiles_n)) / 8);
    {
        const __bf16* P_rows = P + (((tile_r * 256) * K));
        {
            const __bf16* Q_rows = Q + (((tile_c * 256) * K));
            {
                float* D_tile = D + ((((tile_r * 256) * N) + (tile_c * 256)));
                {
                    int __block_id_1 = __block_id_0 % 1;
                    int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
                    __shared__ __bf16 first[32768];
                    __shared__ __bf16 second[32768];
                    float acc[128] = {0};
                    fill_stage_bf16(__block_id_1, __thread_id_1, __smem, first, P_rows, Q_rows, K, 0);
                    __syncthreads();
                    for (int k0 = 0; k0 < K; k0 += 128) {
                        fill_stage_bf16(__block_id_1, __thread_id_1, __smem, second, P_rows, Q_rows, K, (k0 + 64));
                        multiply_stage_bf16(__block_id_1, __thread_id_1, __smem, acc, first);
                        __builtin_amdgcn_sched_group_barrier(0x100, 5, 0);
                        for (int g = 0; g < 7; g++) {
                            __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
                            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                        }
                        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
                        __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(0x100, 5, 0);
                        for (int g = 0; g < 7; g++) {
                            __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
                            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                        }
                        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
                        __syncthreads();
                        fill_stage_bf16(__block_id_1, __thread_id_1, __smem, first, P_rows, Q_rows, K, ((k0 + 128) % K));
                        multiply_stage_bf16(__block_id_1, __thread_id_1, __smem, acc, second);
                        __builtin_amdgcn_sched_group_barrier(0x100, 5, 0);
                        for (int g = 0; g < 7; g++) {
                            __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
                            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                            __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                        }
                        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
                        __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                        __builtin_amdgcn_sched_group_barrier(0x100, 5, 0);
                        for (int g = 0; g < 7; g++) {
                            __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
                            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                        }
                        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
                        __syncthreads();
                    }
                    {
                        float* D_mine = D_tile + (0);
                        int wave = (__thread_id_1 / 64);
                        {
                            int __block_id_2 = __block_id_1;
                            int __thread_id_2 = __thread_id_1 % 64;
                            int lane = __thread_id_2;
                            {
                                int __block_id_3 = __block_id_2;
                                int __thread_id_3 = __thread_id_2 % 1;
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

extern "C" int pipelined_gemm_bf16_launch(const __bf16* P, const __bf16* Q, float* D, int N, int K, int tiles_m, int tiles_n, unsigned grid_blocks, void* stream) {
    if (grid_blocks == 0) return 0;
    pipelined_gemm_bf16<<<dim3(grid_blocks), dim3(512), 0, static_cast<hipStream_t>(stream)>>>(P, Q, D, N, K, tiles_m, tiles_n);
    return static_cast<int>(hipGetLastError());
}
