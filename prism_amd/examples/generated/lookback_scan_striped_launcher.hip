#include <hip/hip_runtime.h>
#include <cstddef>
#include <cstdint>

__device__ uint32_t take_ticket(int __block_id, int __thread_id, char* __smem, uint32_t* counter) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    __shared__ uint32_t ticket;
    if (threadIdx.x == 0) ticket = atomicAdd(counter, 1u);
    __syncthreads();
    return ticket;
}

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

__device__ uint32_t value_of_last_lane(int __block_id, int __thread_id, char* __smem, uint32_t val) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0;
        int __thread_id_1 = __thread_id_0 % 1;
        return __shfl(val, 63, 64);
    }
}

__device__ uint32_t shift_up_in_wavefront(int __block_id, int __thread_id, char* __smem, uint32_t val, uint32_t delta) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0;
        int __thread_id_1 = __thread_id_0 % 1;
        return __shfl_up(val, delta, 64);
    }
}

__global__ void lookback_scan_striped(const uint32_t* x, uint32_t* y, uint32_t* counter, uint64_t* status, int spin_limit) {
    extern __shared__ __align__(128) char __smem[];
    int __block_id_0 = blockIdx.x;
    int __thread_id_0 = __block_id_0 * blockDim.x + threadIdx.x;
    uint32_t tile = take_ticket(__block_id_0, __thread_id_0, __smem, counter);
    {
        const uint32_t* x_tile = x + ((tile * 65536));
        {
            uint32_t* y_tile = y + ((tile * 65536));
            {
                uint64_t* status_blk = status + (0);
                {
                    int __block_id_1 = __block_id_0 % 1;
                    int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
                    __shared__ uint32_t wave_sums[16];
                    int wave = (__thread_id_1 / 64);
                    uint32_t v[64];
                    {
                        const uint32_t* x_wave = x_tile + ((4096 * wave));
                        {
                            uint32_t* my_wave_sum = wave_sums + (wave);
                            {
                                int __block_id_2 = __block_id_1;
                                int __thread_id_2 = __thread_id_1 % 64;
                                uint32_t lane = __thread_id_2;
                                {
                                    const uint32_t* x_mine = x_wave + ((4 * lane));
                                    {
                                        uint32_t* sum_one = my_wave_sum + (0);
                                        {
                                            int __block_id_3 = __block_id_2;
                                            int __thread_id_3 = __thread_id_2 % 1;
                                            for (int j = 0; j < 16; j++) {
                                                for (int e = 0; e < 4; e++) {
                                                    v[((4 * j) + e)] = x_mine[((256 * j) + e)];
                                                }
                                            }
                                            uint32_t carry = 0;
                                            for (int j = 0; j < 16; j++) {
                                                v[((4 * j) + 1)] += v[(4 * j)];
                                                v[((4 * j) + 2)] += v[((4 * j) + 1)];
                                                v[((4 * j) + 3)] += v[((4 * j) + 2)];
                                                uint32_t upto_me = v[((4 * j) + 3)];
                                                uint32_t stride = 1;
                                                while ((stride < 64)) {
                                                    uint32_t got = shift_up_in_wavefront(__block_id_3, __thread_id_3, __smem, upto_me, stride);
                                                    if ((lane >= stride)) {
                                                        upto_me = (got + upto_me);
                                                    }
                                                    stride *= 2;
                                                }
                                                uint32_t ahead = (carry + (upto_me - v[((4 * j) + 3)]));
                                                for (int e = 0; e < 4; e++) {
                                                    v[((4 * j) + e)] += ahead;
                                                }
                                                carry += value_of_last_lane(__block_id_3, __thread_id_3, __smem, upto_me);
                                            }
                                            if ((lane == 63)) {
                                                sum_one[0] = carry;
                                            }
                                        }
                                    }
                                }
                            }
                        }
                    }
                    uint32_t total = 0;
                    __syncthreads();
                    for (int w = 0; w < 16; w++) {
                        total += wave_sums[w];
                    }
                    publish(__block_id_1, __thread_id_1, __smem, status_blk, tile, 1, total);
                    uint32_t before = look_back_wide(__block_id_1, __thread_id_1, __smem, status_blk, tile, spin_limit);
                    publish(__block_id_1, __thread_id_1, __smem, status_blk, tile, 2, (before + total));
                    {
                        uint32_t* y_wave = y_tile + ((4096 * wave));
                        {
                            int __block_id_2 = __block_id_1;
                            int __thread_id_2 = __thread_id_1 % 64;
                            uint32_t lane_out = __thread_id_2;
                            uint32_t earlier_waves = 0;
                            for (int w = 0; w < 16; w++) {
                                if ((w < wave)) {
                                    earlier_waves += wave_sums[w];
                                }
                            }
                            {
                                uint32_t* y_mine = y_wave + ((4 * lane_out));
                                {
                                    int __block_id_3 = __block_id_2;
                                    int __thread_id_3 = __thread_id_2 % 1;
                                    for (int j = 0; j < 16; j++) {
                                        for (int e = 0; e < 4; e++) {
                                            y_mine[((256 * j) + e)] = ((before + earlier_waves) + v[((4 * j) + e)]);
                                        }
                                    }
                                }
                            }
                        }
                    }
                }
            }
        }
    }
}

extern "C" int lookback_scan_striped_launch(const uint32_t* x, uint32_t* y, uint32_t* counter, uint64_t* status, int spin_limit, unsigned grid_blocks, void* stream) {
    if (grid_blocks == 0) return 0;
    lookback_scan_striped<<<dim3(grid_blocks), dim3(1024), 0, static_cast<hipStream_t>(stream)>>>(x, y, counter, status, spin_limit);
    return static_cast<int>(hipGetLastError());
}
