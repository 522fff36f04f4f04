__global__ __launch_bounds__(1024) void pipelined_sgemm(int M, int N, int K, float alpha, const float* A, const float* B, float beta, float* C, int tiles_n) {
    extern __shared__ __align__(128) char __smem[];
    int __block_id_0 = blockIdx.x;
    int __thread_id_0 = __block_id_0 * blockDim.x + threadIdx.x;
    const int per_xcd = (((M / 256) * tiles_n) / 8);
    const int t = (((__block_id_0 % 8) * per_xcd) + (__block_id_0 / 8));
    const int tile_r = ((8 * (t / (8 * tiles_n))) + (t % 8));
    const int tile_c = ((t % (8 * tiles_n)) / 8);
    {
        const float* A_rows = A + (((tile_r * 256) * K));
        {
            const float* B_cols = B + ((tile_c * 256));
            {
                float* C_tile = C + ((((tile_r * 256) * N) + (tile_c * 256)));
                {
                    int __block_id_1 = __block_id_0 % 1;
                    int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
                    __shared__ float first[16384];
                    __shared__ float second[16384];
                    float acc[64] = {0};
                    fill_stage_f32(__block_id_1, __thread_id_1, __smem, first, A_rows, B_cols, N, K, 0);
                    __syncthreads();
                    for (int k0 = 0; k0 < K; k0 += 64) {
                        fill_stage_f32(__block_id_1, __thread_id_1, __smem, second, A_rows, B_cols, N, K, (k0 + 32));
                        multiply_stage_f32(__block_id_1, __thread_id_1, __smem, acc, first);
                        __syncthreads();
                        if (((k0 + 64) < K)) {
                            fill_stage_f32(__block_id_1, __thread_id_1, __smem, first, A_rows, B_cols, N, K, (k0 + 64));
                        }
                        multiply_stage_f32(__block_id_1, __thread_id_1, __smem, acc, second);
                        __syncthreads();
                    }
                    {
                        float* C_mine = C_tile + (0);
                        int wave = (__thread_id_1 / 64);
                        {
                            int __block_id_2 = __block_id_1;
                            int __thread_id_2 = __thread_id_1 % 64;
                            int lane = __thread_id_2;
                            {
                                int __block_id_3 = __block_id_2;
                                int __thread_id_3 = __thread_id_2 % 1;
                                for (int v = 0; v < 16; v++) {
                                    for (int j = 0; j < 4; j++) {
                                        int at = ((((((((32 * (wave / 2)) + (8 * (v / 4))) + (4 * (lane / 32))) + (v % 4)) * N) + (128 * (wave % 2))) + (4 * (lane % 32))) + j);
                                        C_mine[at] = ((alpha * acc[((j * 16) + v)]) + (beta * C_mine[at]));
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
