#include <hip/hip_runtime.h>
#include <cstddef>
#include <cstdint>

__global__ void add_m_blocks(const int* x, int* y, int m, int per_block, int n) {
    extern __shared__ __align__(128) char __smem[];
    int __block_id_0 = blockIdx.x;
    int __thread_id_0 = __block_id_0 * blockDim.x + threadIdx.x;
    int first = (__block_id_0 * per_block);
    {
        const int* x_blk = x + (first);
        {
            int* y_blk = y + (first);
            {
                int __block_id_1 = __block_id_0 % 1;
                int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
                int lane = __thread_id_1;
                {
                    const int* x_one = x_blk + (lane);
                    {
                        int* y_one = y_blk + (lane);
                        {
                            int __block_id_2 = __block_id_1;
                            int __thread_id_2 = __thread_id_1 % 1;
                            if (((first + lane) < n)) {
                                y_one[0] = (x_one[0] + m);
                            }
                        }
                    }
                }
            }
        }
    }
}

extern "C" int add_m_blocks_launch(const int* x, int* y, int m, int per_block, int n, unsigned grid_blocks, void* stream) {
    if (grid_blocks == 0) return 0;
    add_m_blocks<<<dim3(grid_blocks), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(x, y, m, per_block, n);
    return static_cast<int>(hipGetLastError());
}
