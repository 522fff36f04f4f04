#include <hip/hip_runtime.h>
#include <cstddef>
#include <cstdint>

__device__ uint32_t lane_shift_up(int __block_id, int __thread_id, char* __smem, uint32_t val, uint32_t delta) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0;
        int __thread_id_1 = __thread_id_0 % 1;
        return __shfl_up(val, delta, 32);
    }
}

__global__ void row_scan32(const uint32_t* x, uint32_t* y, int rows) {
    extern __shared__ __align__(128) char __smem[];
    int __block_id_0 = blockIdx.x;
    int __thread_id_0 = __block_id_0 * blockDim.x + threadIdx.x;
    int first_row = (__block_id_0 * 8);
    {
        const uint32_t* x_blk = x + ((first_row * 32));
        {
            uint32_t* y_blk = y + ((first_row * 32));
            {
                int __block_id_1 = __block_id_0 % 1;
                int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
                int g = (__thread_id_1 / 32);
                {
                    const uint32_t* x_row = x_blk + ((g * 32));
                    {
                        uint32_t* y_row = y_blk + ((g * 32));
                        {
                            int __block_id_2 = __block_id_1;
                            int __thread_id_2 = __thread_id_1 % 32;
                            uint32_t lane = __thread_id_2;
                            {
                                uint32_t* y_one = y_row + (lane);
                                {
                                    int __block_id_3 = __block_id_2;
                                    int __thread_id_3 = __thread_id_2 % 1;
                                    uint32_t v = 0;
                                    if (((first_row + g) < rows)) {
                                        v = x_row[lane];
                                    }
                                    uint32_t step = 1;
                                    while ((step < 32)) {
                                        uint32_t got = lane_shift_up(__block_id_3, __thread_id_3, __smem, v, step);
                                        if ((lane >= step)) {
                                            v = (got + v);
                                        }
                                        step *= 2;
                                    }
                                    if (((first_row + g) < rows)) {
                                        y_one[0] = v;
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

extern "C" int row_scan32_launch(const uint32_t* x, uint32_t* y, int rows, unsigned grid_blocks, void* stream) {
    if (grid_blocks == 0) return 0;
    row_scan32<<<dim3(grid_blocks), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(x, y, rows);
    return static_cast<int>(hipGetLastError());
}
