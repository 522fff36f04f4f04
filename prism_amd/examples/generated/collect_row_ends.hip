__device__ void collect_row_ends(int __block_id, int __thread_id, char* __smem, const uint32_t* scanned, uint32_t* ends) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0 % 1;
        int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
        uint32_t t = __thread_id_1;
        {
            uint32_t* end_one = ends + (t);
            {
                int __block_id_2 = __block_id_1;
                int __thread_id_2 = __thread_id_1 % 1;
                if ((t < 16)) {
                    end_one[0] = scanned[((64 * t) + 63)];
                }
            }
        }
    }
    return;
}
