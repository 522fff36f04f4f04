__device__ void publish(int __block_id, int __thread_id, char* __smem, uint64_t* status, uint32_t tile, uint32_t flag, uint32_t value) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0 % 1;
        int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
        if (threadIdx.x == 0)
            __hip_atomic_store(&status[tile], (static_cast<uint64_t>(flag) << 32) | value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    return;
}
