template<int BM, int BN, int BK, int TM, int TN>
__global__ __launch_bounds__((BM * BN) / (TM * TN)) void thread_tile_sgemm(int M, int N, int K, float alpha, const float* A, const float* B, float beta, float* C, int tiles_n) {
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
                    const int threads = ((BM * BN) / (TM * TN));
                    const int out_r = (t / (BN / TN));
                    const int out_c = (t % (BN / TN));
                    float acc[16] = {0};
                    float a_reg[4] = {0};
                    float b_reg[4] = {0};
                    for (int k0 = 0; k0 < K; k0 += BK) {
                        {
                            float* a_mine = a_lds + (0);
                            {
                                float* b_mine = b_lds + (0);
                                {
                                    int __block_id_2 = __block_id_1;
                                    int __thread_id_2 = __thread_id_1 % 1;
                                    for (int e = t; e < (BM * BK); e += threads) {
                                        a_mine[e] = A_rows[((((e / BK) * K) + k0) + (e % BK))];
                                    }
                                    for (int e = t; e < (BK * BN); e += threads) {
                                        b_mine[e] = B_cols[(((k0 + (e / BN)) * N) + (e % BN))];
                                    }
                                    __syncthreads();
                                    for (int kk = 0; kk < BK; kk++) {
                                        for (int i = 0; i < TM; i++) {
                                            a_reg[i] = a_lds[((((out_r * TM) + i) * BK) + kk)];
                                        }
                                        for (int j = 0; j < TN; j++) {
                                            b_reg[j] = b_lds[(((kk * BN) + (out_c * TN)) + j)];
                                        }
                                        for (int i = 0; i < TM; i++) {
                                            for (int j = 0; j < TN; j++) {
                                                acc[((i * TN) + j)] += (a_reg[i] * b_reg[j]);
                                            }
                                        }
                                    }
                                }
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
