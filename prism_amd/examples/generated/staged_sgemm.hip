template<int BM, int BN, int BK, int TM, int TN, int THREADS>
__global__ __launch_bounds__(THREADS) void staged_sgemm(int M, int N, int K, float alpha, const float* A, const float* B, float beta, float* C, int tiles_n) {
    extern __shared__ __align__(128) char __smem[];
    int __block_id_0 = blockIdx.x;
    int __thread_id_0 = __block_id_0 * blockDim.x + threadIdx.x;
    const int tile_r = (__block_id_0 / tiles_n);
    const int tile_c = (__block_id_0 % tiles_n);
    {
        const float* A_rows = A + (((tile_r * BM) * K));
        {
            const float* B_cols = B + ((tile_c * BN));
            {
                float* C_tile = C + ((((tile_r * BM) * N) + (tile_c * BN)));
                {
                    int __block_id_1 = __block_id_0 % 1;
                    int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
                    float (&a_lds)[1024] = *((float (*)[1024])(__smem + 0));
                    float (&b_lds)[1024] = *((float (*)[1024])(__smem + 4096));
                    const int t = __thread_id_1;
                    const int out_r = (t / (BN / TN));
                    const int out_c = (t % (BN / TN));
                    float acc[16] = {0};
                    for (int k0 = 0; k0 < K; k0 += BK) {
                        {
                            const float* A_now = A_rows + (k0);
                            {
                                const float* B_now = B_cols + ((k0 * N));
                                stage_tiles<BM, BN, BK, THREADS>(__block_id_1, __thread_id_1, __smem, N, K, A_now, B_now, a_lds, b_lds);
                                __syncthreads();
                                multiply_tiles<BM, BN, BK, TM, TN>(__block_id_1, __thread_id_1, __smem, acc, a_lds, b_lds, out_r, out_c);
                            }
                        }
                        __syncthreads();
                    }
                    {
                        float* C_mine = C_tile + ((((out_r * TM) * N) + (out_c * TN)));
                        {
                            int __block_id_2 = __block_id_1;
                            int __thread_id_2 = __thread_id_1 % 1;
                            for (int i = 0; i < TM; i++) {
                                for (int j = 0; j < TN; j++) {
                                    C_mine[((i * N) + j)] = ((alpha * acc[((i * TN) + j)]) + (beta * C_mine[((i * N) + j)]));
                                }
                            }
                        }
                    }
                }
            }
        }
    }
}
