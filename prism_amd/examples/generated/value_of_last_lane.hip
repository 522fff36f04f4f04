__device__ uint32_t value_of_last_lane(int __block_id, int __thread_id, char* __smem, uint32_t val) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0;
        int __thread_id_1 = __thread_id_0 % 1;
        return __shfl(val, 63, 64);
    }
}
