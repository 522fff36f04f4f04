__device__ uint32_t look_back_wide(int __block_id, int __thread_id, char* __smem, uint64_t* status, uint32_t tile, int spin_limit) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0 % 1;
        int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
        __shared__ uint32_t before;
        if (threadIdx.x < 64) {
            uint32_t sum = 0;
            int nearest = static_cast<int>(tile) - 1, spins = 0;
            bool done = false;
            while (!done) {
                const int id = nearest - static_cast<int>(threadIdx.x);
                for (;;) {
                    const uint64_t word = id >= 0 ? __hip_atomic_load(&status[id], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                                                  : (static_cast<uint64_t>(2) << 32);
                    const uint64_t prefixes = __ballot((word >> 32) == 2), missing = __ballot((word >> 32) == 0);
                    const int first = prefixes ? __ffsll(static_cast<unsigned long long>(prefixes)) - 1 : 64;
                    const uint64_t wanted = first >= 63 ? ~0ull : ((1ull << (first + 1)) - 1);
                    if ((missing & wanted) == 0 || ++spins > spin_limit) {
                        uint32_t part = static_cast<int>(threadIdx.x) <= first ? static_cast<uint32_t>(word) : 0u;
                        for (int o = 32; o > 0; o >>= 1) part += __shfl_xor(part, o, 64);
                        sum += part;
                        done = first < 64 || spins > spin_limit;
                        nearest -= 64;
                        break;
                    }
                    __builtin_amdgcn_s_sleep(1);
                }
            }
            if (threadIdx.x == 0) before = sum;
        }
        __syncthreads();
        return before;
    }
}
