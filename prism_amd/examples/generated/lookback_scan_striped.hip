__global__ void lookback_scan_striped(const uint32_t* x, uint32_t* y, uint32_t* counter, uint64_t* status, int spin_limit) {
    extern __shared__ __align__(128) char __smem[];
    int __block_id_0 = blockIdx.x;
    int __thread_id_0 = __block_id_0 * blockDim.x + threadIdx.x;
    uint32_t tile = take_ticket(__block_id_0, __thread_id_0, __smem, counter);
    {
        const uint32_t* x_tile = x + ((tile * 65536));
        {
            uint32_t* y_tile = y + ((tile * 65536));
            {
                uint64_t* status_blk = status + (0);
                {
                    int __block_id_1 = __block_id_0 % 1;
                    int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
                    __shared__ uint32_t wave_sums[16];
                    int wave = (__thread_id_1 / 64);
                    uint32_t v[64];
                    {
                        const uint32_t* x_wave = x_tile + ((4096 * wave));
                        {
                            uint32_t* my_wave_sum = wave_sums + (wave);
                            {
                                int __block_id_2 = __block_id_1;
                                int __thread_id_2 = __thread_id_1 % 64;
                                uint32_t lane = __thread_id_2;
                                {
                                    const uint32_t* x_mine = x_wave + ((4 * lane));
                                    {
                                        uint32_t* sum_one = my_wave_sum + (0);
                                        {
                                            int __block_id_3 = __block_id_2;
                                            int __thread_id_3 = __thread_id_2 % 1;
                                            for (int j = 0; j < 16; j++) {
                                                for (int e = 0; e < 4; e++) {
                                                    v[((4 * j) + e)] = x_mine[((256 * j) + e)];
                                                }
                                            }
                                            uint32_t carry = 0;
                                            for (int j = 0; j < 16; j++) {
                                                v[((4 * j) + 1)] += v[(4 * j)];
                                                v[((4 * j) + 2)] += v[((4 * j) + 1)];
                                                v[((4 * j) + 3)] += v[((4 * j) + 2)];
                                                uint32_t upto_me = v[((4 * j) + 3)];
                                                uint32_t stride = 1;
                                                while ((stride < 64)) {
                                                    uint32_t got = shift_up_in_wavefront(__block_id_3, __thread_id_3, __smem, upto_me, stride);
                                                    if ((lane >= stride)) {
                                                        upto_me = (got + upto_me);
                                                    }
                                                    stride *= 2;
                                                }
                                                uint32_t ahead = (carry + (upto_me - v[((4 * j) + 3)]));
                                                for (int e = 0; e < 4; e++) {
                                                    v[((4 * j) + e)] += ahead;
                                                }
                                                carry += value_of_last_lane(__block_id_3, __thread_id_3, __smem, upto_me);
                                            }
                                            if ((lane == 63)) {
                                                sum_one[0] = carry;
                                            }
                                        }
                                    }
                                }
                            }
                        }
                    }
                    uint32_t total = 0;
                    __syncthreads();
                    for (int w = 0; w < 16; w++) {
                        total += wave_sums[w];
                    }
                    publish(__block_id_1, __thread_id_1, __smem, status_blk, tile, 1, total);
                    uint32_t before = look_back_wide(__block_id_1, __thread_id_1, __smem, status_blk, tile, spin_limit);
                    publish(__block_id_1, __thread_id_1, __smem, status_blk, tile, 2, (before + total));
                    {
                        uint32_t* y_wave = y_tile + ((4096 * wave));
                        {
                            int __block_id_2 = __block_id_1;
                            int __thread_id_2 = __thread_id_1 % 64;
                            uint32_t lane_out = __thread_id_2;
                            uint32_t earlier_waves = 0;
                            for (int w = 0; w < 16; w++) {
                                if ((w < wave)) {
                                    earlier_waves += wave_sums[w];
                                }
                            }
                            {
                                uint32_t* y_mine = y_wave + ((4 * lane_out));
                                {
                                    int __block_id_3 = __block_id_2;
                                    int __thread_id_3 = __thread_id_2 % 1;
                                    for (int j = 0; j < 16; j++) {
                                        for (int e = 0; e < 4; e++) {
                                            y_mine[((256 * j) + e)] = ((before + earlier_waves) + v[((4 * j) + e)]);
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
