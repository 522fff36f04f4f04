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
