__global__ void lookback_scan_wide(const uint32_t* x, uint32_t* y, uint32_t* counter, uint64_t* status, int spin_limit) {
    extern __shared__ __align__(128) char __smem[];
    int __block_id_0 = blockIdx.x;
    int __thread_id_0 = __block_id_0 * blockDim.x + threadIdx.x;
    uint32_t tile = take_ticket(__block_id_0, __thread_id_0, __smem, counter);
    {
        const uint32_t* x_tile = x + ((tile * 4096));
        {
            uint32_t* y_tile = y + ((tile * 4096));
            {
                uint64_t* status_blk = status + (0);
                {
                    int __block_id_1 = __block_id_0 % 1;
                    int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
                    __shared__ uint32_t wave_sums[4];
                    int t = __thread_id_1;
                    int wave = (__thread_id_1 / 64);
                    uint32_t v[16];
                    {
                        const uint32_t* x_mine = x_tile + ((16 * t));
                        {
                            int __block_id_2 = __block_id_1;
                            int __thread_id_2 = __thread_id_1 % 1;
                            for (int i = 0; i < 16; i++) {
                                v[i] = x_mine[i];
                            }
                            for (int i = 1; i < 16; i++) {
                                v[i] += v[(i - 1)];
                            }
                        }
                    }
                    uint32_t upto_me = v[15];
                    {
                        uint32_t* my_wave_sum = wave_sums + (wave);
                        {
                            int __block_id_2 = __block_id_1;
                            int __thread_id_2 = __thread_id_1 % 64;
                            uint32_t lane = __thread_id_2;
                            {
                                uint32_t* sum_one = my_wave_sum + (0);
                                {
                                    int __block_id_3 = __block_id_2;
                                    int __thread_id_3 = __thread_id_2 % 1;
                                    uint32_t stride = 1;
                                    while ((stride < 64)) {
                                        uint32_t got = shift_up_in_wavefront(__block_id_3, __thread_id_3, __smem, upto_me, stride);
                                        if ((lane >= stride)) {
                                            upto_me = (got + upto_me);
                                        }
                                        stride *= 2;
                                    }
                                    if ((lane == 63)) {
                                        sum_one[0] = upto_me;
                                    }
                                }
                            }
                        }
                    }
                    __syncthreads();
                    uint32_t total = (((wave_sums[0] + wave_sums[1]) + wave_sums[2]) + wave_sums[3]);
                    publish(__block_id_1, __thread_id_1, __smem, status_blk, tile, 1, total);
                    uint32_t before = look_back_wide(__block_id_1, __thread_id_1, __smem, status_blk, tile, spin_limit);
                    publish(__block_id_1, __thread_id_1, __smem, status_blk, tile, 2, (before + total));
                    {
                        uint32_t* y_mine = y_tile + ((16 * t));
                        {
                            int __block_id_2 = __block_id_1;
                            int __thread_id_2 = __thread_id_1 % 64;
                            uint32_t earlier_waves = 0;
                            for (int w = 0; w < 4; w++) {
                                if ((w < wave)) {
                                    earlier_waves += wave_sums[w];
                                }
                            }
                            {
                                int __block_id_3 = __block_id_2;
                                int __thread_id_3 = __thread_id_2 % 1;
                                uint32_t base = ((before + earlier_waves) + (upto_me - v[15]));
                                for (int i = 0; i < 16; i++) {
                                    y_mine[i] = (base + v[i]);
                                }
                            }
                        }
                    }
                }
            }
        }
    }
}
