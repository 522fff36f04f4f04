__device__ void write_back(int __block_id, int __thread_id, char* __smem, uint32_t* y_tile, const uint32_t* scanned, const uint32_t* upto, uint32_t before) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0 % 1;
        int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
        int t = __thread_id_1;
        {
            uint32_t* y_mine = y_tile + (t);
            {
                int __block_id_2 = __block_id_1;
                int __thread_id_2 = __thread_id_1 % 1;
                for (int k = 0; k < 4; k++) {
                    int el = (t + (256 * k));
                    int row = (el / 64);
                    uint32_t base = before;
                    if ((row > 0)) {
                        base = (before + upto[(row - 1)]);
                    }
                    y_mine[(256 * k)] = (base + scanned[el]);
                }
            }
        }
    }
    return;
}
