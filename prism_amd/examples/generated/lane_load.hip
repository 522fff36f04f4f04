__device__ void lane_load(int __block_id, int __thread_id, char* __smem, const int* src, int* dst, int items) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0;
        int __thread_id_1 = __thread_id_0 % 1;
        for (int i = 0; i < items; i++) {
            dst[i] = src[i];
        }
    }
}
