#include <hip/hip_runtime.h>
#include <cstddef>
#include <cstdint>

__global__ void gather_columns(const int* x, int* y, int rows, int cols) {
    extern __shared__ __align__(128) char __smem[];
    int __block_id_0 = blockIdx.x;
    int __thread_id_0 = __block_id_0 * blockDim.x + threadIdx.x;
    int c = __thread_id_0;
    {
        int* mine = y + ((c * rows));
        {
            int __block_id_1 = __block_id_0 % 1;
            int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
            {
                int __block_id_2 = __block_id_1;
                int __thread_id_2 = __thread_id_1 % 1;
                if ((c < cols)) {
                    mine[0] = x[((0 * cols) + c)];
                    for (int r = 0; r < (rows - 1); r++) {
                        mine[(r + 1)] = x[(((r + 1) * cols) + c)];
                    }
                }
            }
        }
    }
}

extern "C" int gather_columns_launch(const int* x, int* y, int rows, int cols, unsigned grid_blocks, void* stream) {
    if (grid_blocks == 0) return 0;
    gather_columns<<<dim3(grid_blocks), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(x, y, rows, cols);
    return static_cast<int>(hipGetLastError());
}
