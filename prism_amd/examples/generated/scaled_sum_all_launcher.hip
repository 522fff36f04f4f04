#include <hip/hip_runtime.h>
#include <cstddef>
#include <cstdint>

__device__ float scaled_sum(int __block_id, int __thread_id, char* __smem, float a, float b, float s) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    return (s * (a + b));
}

__global__ void scaled_sum_all(const float* x, float* y, float s, int n) {
    extern __shared__ __align__(128) char __smem[];
    int __block_id_0 = blockIdx.x;
    int __thread_id_0 = __block_id_0 * blockDim.x + threadIdx.x;
    int i = __thread_id_0;
    {
        float* y_one = y + (i);
        {
            int __block_id_1 = __block_id_0 % 1;
            int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
            {
                int __block_id_2 = __block_id_1;
                int __thread_id_2 = __thread_id_1 % 1;
                if ((i < n)) {
                    y_one[0] = scaled_sum(__block_id_2, __thread_id_2, __smem, x[i], y_one[0], s);
                }
            }
        }
    }
}

extern "C" int scaled_sum_all_launch(const float* x, float* y, float s, int n, unsigned grid_blocks, void* stream) {
    if (grid_blocks == 0) return 0;
    scaled_sum_all<<<dim3(grid_blocks), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(x, y, s, n);
    return static_cast<int>(hipGetLastError());
}
