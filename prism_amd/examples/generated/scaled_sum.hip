__device__ float scaled_sum(int __block_id, int __thread_id, char* __smem, float a, float b, float s) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    return (s * (a + b));
}
