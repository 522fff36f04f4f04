__global__ __launch_bounds__(256) void mfma_tile_sgemm(int M, int N, int K, float alpha, const float* A, const float* B, float beta, float* C, int tiles_n) {
    extern __shared__ __align__(128) char __smem[];
    int __block_id_0 = blockIdx.x;
    int __thread_id_0 = __block_id_0 * blockDim.x + threadIdx.x;
    const int tile_r = (__block_id_0 / tiles_n);
    const int tile_c = (__block_id_0 % tiles_n);
    {
        const float* A_rows = A + (((tile_r * 64) * K));
        {
            const float* B_cols = B + ((tile_c * 64));
            {
                float* C_tile = C + ((((tile_r * 64) * N) + (tile_c * 64)));
                {
                    int __block_id_1 = __block_id_0 % 1;
                    int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
                    __shared__ float a_lds[512];
                    __shared__ float b_lds[512];
                    const int t = __thread_id_1;
                    const int wave = (__thread_id_1 / 64);
                    const int corner_r = ((wave / 2) * 32);
                    const int corner_c = ((wave % 2) * 32);
                    {
                        float* a_mine = a_lds + (0);
                        {
                            float* b_mine = b_lds + (0);
                            {
                                float* C_mine = C_tile + (0);
                                {
                                    int __block_id_2 = __block_id_1;
                                    int __thread_id_2 = __thread_id_1 % 64;
                                    const int lane = __thread_id_2;
                                    const int r = (lane % 32);
                                    const int q = (lane / 32);
                                    float acc[16] = {0};
                                    {
                                        int __block_id_3 = __block_id_2;
                                        int __thread_id_3 = __thread_id_2 % 1;
                                        for (int k0 = 0; k0 < K; k0 += 8) {
                                            for (int e = t; e < 512; e += 256) {
                                                a_mine[(((e % 8) * 64) + (e / 8))] = A_rows[((((e / 8) * K) + k0) + (e % 8))];
                                                b_mine[e] = B_cols[(((k0 + (e / 64)) * N) + (e % 64))];
                                            }
                                            __syncthreads();
                                            for (int kk = 0; kk < 8; kk += 2) {
                                                {
                                                    typedef float __acc_t __attribute__((ext_vector_type(16)));
                                                    __acc_t __acc = {acc[0], acc[1], acc[2], acc[3], acc[4], acc[5], acc[6], acc[7], acc[8], acc[9], acc[10], acc[11], acc[12], acc[13], acc[14], acc[15]};
                                                    __acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a_lds[((((kk + q) * 64) + corner_r) + r)], b_lds[((((kk + q) * 64) + corner_c) + r)], __acc, 0, 0, 0);
                                                    acc[0] = __acc[0];
                                                    acc[1] = __acc[1];
                                                    acc[2] = __acc[2];
                                                    acc[3] = __acc[3];
                                                    acc[4] = __acc[4];
                                                    acc[5] = __acc[5];
                                                    acc[6] = __acc[6];
                                                    acc[7] = __acc[7];
                                                    acc[8] = __acc[8];
                                                    acc[9] = __acc[9];
                                                    acc[10] = __acc[10];
                                                    acc[11] = __acc[11];
                                                    acc[12] = __acc[12];
                                                    acc[13] = __acc[13];
                                                    acc[14] = __acc[14];
                                                    acc[15] = __acc[15];
                                                }
                                            }
                                            __syncthreads();
                                        }
                                        for (int v = 0; v < 16; v++) {
                                            C_mine[((((((corner_r + (8 * (v / 4))) + (4 * q)) + (v % 4)) * N) + corner_c) + r)] = ((alpha * acc[v]) + (beta * C_mine[((((((corner_r + (8 * (v / 4))) + (4 * q)) + (v % 4)) * N) + corner_c) + r)]));
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
