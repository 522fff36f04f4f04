__global__ void one_bf16_mfma_per_wavefront(const __bf16* P, const __bf16* Q, float* D, int M, int N, int K) {
    extern __shared__ __align__(128) char __smem[];
    int __block_id_0 = blockIdx.x;
    int __thread_id_0 = __block_id_0 * blockDim.x + threadIdx.x;
    const int tiles_n = (N / 16);
    const int w = (__thread_id_0 / 64);
    const int tile_r = (w / tiles_n);
    const int tile_c = (w % tiles_n);
    {
        const __bf16* P_rows = P + (((tile_r * 16) * K));
        {
            const __bf16* Q_rows = Q + (((tile_c * 16) * K));
            {
                float* D_tile = D + ((((tile_r * 16) * N) + (tile_c * 16)));
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
                            for (int k0 = 0; k0 < K; k0 += 32) {
                                float4 a = reinterpret_cast<const float4 *>(&P_rows[(((r * K) + k0) + (8 * q))])[0];
                                float4 b = reinterpret_cast<const float4 *>(&Q_rows[(((r * K) + k0) + (8 * q))])[0];
                                {
                                    typedef float __acc_t __attribute__((ext_vector_type(4)));
                                    __acc_t __acc = {c0, c1, c2, c3};
                                    typedef __bf16 __packet_t __attribute__((ext_vector_type(8)));
                                    __acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(__packet_t, a), __builtin_bit_cast(__packet_t, b), __acc, 0, 0, 0);
                                    c0 = __acc[0];
                                    c1 = __acc[1];
                                    c2 = __acc[2];
                                    c3 = __acc[3];
                                }
                            }
                        }
                        {
                            float* D_mine = D_tile + ((((4 * q) * N) + r));
                            {
                                int __block_id_3 = __block_id_2;
                                int __thread_id_3 = __thread_id_2 % 1;
                                if ((w < ((M / 16) * tiles_n))) {
                                    D_mine[(0 * N)] = c0;
                                    D_mine[(1 * N)] = c1;
                                    D_mine[(2 * N)] = c2;
                                    D_mine[(3 * N)] = c3;
                                }
                            }
                        }
                    }
                }
            }
        }
    }
}
