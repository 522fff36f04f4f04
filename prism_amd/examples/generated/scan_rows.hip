__device__ void scan_rows(int __block_id, int __thread_id, char* __smem, const uint32_t* x_tile, uint32_t* scanned) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0 % 1;
        int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
        int wave = (__thread_id_1 / 64);
        for (int i = 0; i < 4; i++) {
            {
                const uint32_t* x_row = x_tile + (((wave + (4 * i)) * 64));
                {
                    uint32_t* s_row = scanned + (((wave + (4 * i)) * 64));
                    {
                        int __block_id_2 = __block_id_1;
                        int __thread_id_2 = __thread_id_1 % 64;
                        uint32_t lane = __thread_id_2;
                        {
                            uint32_t* s_one = s_row + (lane);
                            {
                                int __block_id_3 = __block_id_2;
                                int __thread_id_3 = __thread_id_2 % 1;
                                uint32_t v = x_row[lane];
                                uint32_t stride = 1;
                                while ((stride < 64)) {
                                    uint32_t got = shift_up_in_wavefront(__block_id_3, __thread_id_3, __smem, v, stride);
                                    if ((lane >= stride)) {
                                        v = (got + v);
                                    }
                                    stride *= 2;
                                }
                                s_one[0] = v;
                            }
                        }
                    }
                }
            }
        }
    }
    return;
}
