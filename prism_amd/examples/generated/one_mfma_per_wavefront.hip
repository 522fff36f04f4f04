__global__ void one_mfma_per_wavefront(const float* A, const float* B, float* C, int M, int N, int K) {
    extern __shared__ __align__(128) char __smem[];
    int __block_id_0 = blockIdx.x;
    int __thread_id_0 = __block_id_0 * blockDim.x + threadIdx.x;
    const int tiles_n = (N / 16);
    const int w = (__thread_id_0 / 64);
    const int tile_r = (w / tiles_n);
    const int tile_c = (w % tiles_n);
    {
        const float* A_rows = A + (((tile_r * 16) * K));
        {
            const float* B_cols = B + ((tile_c * 16));
            {
                float* C_tile = C + ((((tile_r * 16) * N) + (tile_c * 16)));
                {
                    int __block_id_1 = __block_id_0 % 1;
                    int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
                    {
                        int __block_id_2 = __block_id_1;
                        int __thread_id_2 = __thread_id_1 % 64;
                        const int lane = __thread_id_2;
                        const int r = (lane % 16);
                        const int q = (lane / 16);
                        float c0 = 0;
                        float c1 = 0;
                        float c2 = 0;
                        float c3 = 0;
                        if ((w < ((M / 16) * tiles_n))) {
                            for (int k0 = 0; k0 < K; k0 += 4) {
                                {
                                    typedef float __acc_t __attribute__((ext_vector_type(4)));
                                    __acc_t __acc = {c0, c1, c2, c3};
                                    __acc = __builtin_amdgcn_mfma_f32_16x16x4f32(A_rows[(((r * K) + k0) + q)], B_cols[(((k0 + q) * N) + r)], __acc, 0, 0, 0);
                                    c0 = __acc[0];
                                    c1 = __acc[1];
                                    c2 = __acc[2];
                                    c3 = __acc[3];
                                }
                            }
                        }
                        {
                            float* C_mine = C_tile + ((((4 * q) * N) + r));
                            {
                                int __block_id_3 = __block_id_2;
                                int __thread_id_3 = __thread_id_2 % 1;
                                if ((w < ((M / 16) * tiles_n))) {
                                    C_mine[(0 * N)] = c0;
                                    C_mine[(1 * N)] = c1;
                                    C_mine[(2 * N)] = c2;
                                    C_mine[(3 * N)] = c3;
                                }
                            }
                        }
                    }
                }
            }
        }
    }
}
