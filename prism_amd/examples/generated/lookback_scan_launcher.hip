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

__device__ uint32_t shift_up_in_wavefront(int __block_id, int __thread_id, char* __smem, uint32_t val, uint32_t delta) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0;
        int __thread_id_1 = __thread_id_0 % 1;
        return __shfl_up(val, delta, 64);
    }
}

__global__ void lookback_scan(const uint32_t* x, uint32_t* y, uint32_t* counter, uint64_t* status, int spin_limit) {
    extern __shared__ __align__(128) char __smem[];
    int __block_id_0 = blockIdx.x;
    int __thread_id_0 = __block_id_0 * blockDim.x + threadIdx.x;
    uint32_t tile = take_ticket(__block_id_0, __thread_id_0, __smem, counter);
    {
        const uint32_t* x_tile = x + ((tile * 1024));
        {
            uint32_t* y_tile = y + ((tile * 1024));
            {
                uint64_t* status_blk = status + (0);
                {
                    int __block_id_1 = __block_id_0 % 1;
                    int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
                    __shared__ uint32_t scanned[1024];
                    __shared__ uint32_t ends[16];
                    __shared__ uint32_t upto[16];
                    int wave = (__thread_id_1 / 64);
                    for (int i = 0; i < 4; i++) {
                        {
                            const uint32_t* x_row = x_tile + (((wave + (4 * i)) * 64));
                            {
                                uint32_t* s_row = scanned + (((wave + (4 * i)) * 64));
                                {
                                    uint32_t* row_end = ends + ((wave + (4 * i)));
                                    {
                                        int __block_id_2 = __block_id_1;
                                        int __thread_id_2 = __thread_id_1 % 64;
                                        uint32_t lane = __thread_id_2;
                                        {
                                            uint32_t* s_one = s_row + (lane);
                                            {
                                                uint32_t* end_one = row_end + (0);
                                                {
                                                    int __block_id_3 = __block_id_2;
                                                    int __thread_id_3 = __thread_id_2 % 1;
                                                    uint32_t v = x_row[lane];
                                                    uint32_t stride = 1;
                                                    while ((stride < 64)) {
                                                        uint32_t got = shift_up_in_wavefront(__block_id_3, __thread_id_3, __smem, v, stride);
                                                        if ((lane >= stride)) {
                                                            v = (got + v);
                                                        }
                                                        stride *= 2;
                                                    }
                                                    s_one[0] = v;
                                                    if ((lane == 63)) {
                                                        end_one[0] = v;
                                                    }
                                                }
                                            }
                                        }
                                    }
                                }
                            }
                        }
                    }
                    {
                        uint32_t* upto_wave = upto + (0);
                        {
                            int __block_id_2 = __block_id_1;
                            int __thread_id_2 = __thread_id_1 % 64;
                            uint32_t lane16 = __thread_id_2;
                            {
                                uint32_t* upto_one = upto_wave + (lane16);
                                {
                                    int __block_id_3 = __block_id_2;
                                    int __thread_id_3 = __thread_id_2 % 1;
                                    __syncthreads();
                                    if ((wave == 0)) {
                                        uint32_t e = 0;
                                        if ((lane16 < 16)) {
                                            e = ends[lane16];
                                        }
                                        uint32_t step = 1;
                                        while ((step < 16)) {
                                            uint32_t below = shift_up_in_wavefront(__block_id_3, __thread_id_3, __smem, e, step);
                                            if ((lane16 >= step)) {
                                                e = (below + e);
                                            }
                                            step *= 2;
                                        }
                                        if ((lane16 < 16)) {
                                            upto_one[0] = e;
                                        }
                                    }
                                }
                            }
                        }
                    }
                    __syncthreads();
                    uint32_t total = upto[15];
                    publish(__block_id_1, __thread_id_1, __smem, status_blk, tile, 1, total);
                    uint32_t before = look_back(__block_id_1, __thread_id_1, __smem, status_blk, tile, spin_limit);
                    publish(__block_id_1, __thread_id_1, __smem, status_blk, tile, 2, (before + total));
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
            }
        }
    }
}

extern "C" int lookback_scan_launch(const uint32_t* x, uint32_t* y, uint32_t* counter, uint64_t* status, int spin_limit, unsigned grid_blocks, void* stream) {
    if (grid_blocks == 0) return 0;
    lookback_scan<<<dim3(grid_blocks), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(x, y, counter, status, spin_limit);
    return static_cast<int>(hipGetLastError());
}
