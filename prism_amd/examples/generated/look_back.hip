__device__ uint32_t look_back(int __block_id, int __thread_id, char* __smem, uint64_t* status, uint32_t tile, int spin_limit) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0 % 1;
        int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
        __shared__ uint32_t before;
        if (threadIdx.x == 0) {
            uint32_t sum = 0;
            for (int id = static_cast<int>(tile) - 1; id >= 0; --id) {
                uint64_t word = 0;
                for (int spins = 0; spins < spin_limit; ++spins) {
                    word = __hip_atomic_load(&status[id], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                    if (word >> 32) break;
                    __builtin_amdgcn_s_sleep(1);
                }
                sum += static_cast<uint32_t>(word);
                if ((word >> 32) != 1) break;  // an inclusive prefix ends the walk (and so does a poll that ran out)
            }
            before = sum;
        }
        __syncthreads();
        return before;
    }
}
