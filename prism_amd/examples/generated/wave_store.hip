__device__ void wave_store(int __block_id, int __thread_id, char* __smem, const int* src, int* dst, int items) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0;
        int __thread_id_1 = __thread_id_0 % 64;
        int lane = __thread_id_1;
        {
            int* mine = dst + ((lane * items));
            {
                int __block_id_2 = __block_id_1;
                int __thread_id_2 = __thread_id_1 % 1;
                lane_store(__block_id_2, __thread_id_2, __smem, src, mine, items);
            }
        }
    }
}
