__global__ void add_m_by_wavefronts(const int* x, int* y, int m, int wavefronts) {
    extern __shared__ __align__(128) char __smem[];
    int __block_id_0 = blockIdx.x;
    int __thread_id_0 = __block_id_0 * blockDim.x + threadIdx.x;
    int w = (__thread_id_0 / 64);
    {
        const int* x_wave = x + ((w * 256));
        {
            int* y_wave = y + ((w * 256));
            {
                int __block_id_1 = __block_id_0 % 1;
                int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
                {
                    int __block_id_2 = __block_id_1;
                    int __thread_id_2 = __thread_id_1 % 64;
                    int held[4];
                    if ((w < wavefronts)) {
                        wave_load(__block_id_2, __thread_id_2, __smem, x_wave, held, 4);
                        for (int i = 0; i < 4; i++) {
                            held[i] += m;
                        }
                        wave_store(__block_id_2, __thread_id_2, __smem, held, y_wave, 4);
                    }
                }
            }
        }
    }
}
