#include <hip/hip_runtime.h>
#include <cstddef>
#include <cstdint>

__device__ void lane_load(int __block_id, int __thread_id, char* __smem, const int* src, int* dst, int items) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0;
        int __thread_id_1 = __thread_id_0 % 1;
        for (int i = 0; i < items; i++) {
            dst[i] = src[i];
        }
    }
}

__device__ void wave_load(int __block_id, int __thread_id, char* __smem, const int* src, int* dst, int items) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0;
        int __thread_id_1 = __thread_id_0 % 64;
        int lane = __thread_id_1;
        {
            const int* mine = src + ((lane * items));
            {
                int __block_id_2 = __block_id_1;
                int __thread_id_2 = __thread_id_1 % 1;
                lane_load(__block_id_2, __thread_id_2, __smem, mine, dst, items);
            }
        }
    }
}

__device__ void lane_store(int __block_id, int __thread_id, char* __smem, const int* src, int* dst, int items) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0;
        int __thread_id_1 = __thread_id_0 % 1;
        for (int i = 0; i < items; i++) {
            dst[i] = src[i];
        }
    }
}

__device__ void wave_store(int __block_id, int __thread_id, char* __smem, const int* src, int* dst, int items) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0;
        int __thread_id_1 = __thread_id_0 % 64;
        int lane = __thread_id_1;
        {
            int* mine = dst + ((lane * items));
            {
                int __block_id_2 = __block_id_1;
                int __thread_id_2 = __thread_id_1 % 1;
                lane_store(__block_id_2, __thread_id_2, __smem, src, mine, items);
            }
        }
    }
}

__global__ void add_m_by_wavefronts(const int* x, int* y, int m, int wavefronts) {
    extern __shared__ __align__(128) char __smem[];
    int __block_id_0 = blockIdx.x;
    int __thread_id_0 = __block_id_0 * blockDim.x + threadIdx.x;
    int w = (__thread_id_0 / 64);
    {
        const int* x_wave = x + ((w * 256));
        {
            int* y_wave = y + ((w * 256));
            {
                int __block_id_1 = __block_id_0 % 1;
                int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
                {
                    int __block_id_2 = __block_id_1;
                    int __thread_id_2 = __thread_id_1 % 64;
                    int held[4];
                    if ((w < wavefronts)) {
                        wave_load(__block_id_2, __thread_id_2, __smem, x_wave, held, 4);
                        for (int i = 0; i < 4; i++) {
                            held[i] += m;
                        }
                        wave_store(__block_id_2, __thread_id_2, __smem, held, y_wave, 4);
                    }
                }
            }
        }
    }
}

extern "C" int add_m_by_wavefronts_launch(const int* x, int* y, int m, int wavefronts, unsigned grid_blocks, void* stream) {
    if (grid_blocks == 0) return 0;
    add_m_by_wavefronts<<<dim3(grid_blocks), dim3(256), 0, static_cast<hipStream_t>(stream)>>>(x, y, m, wavefronts);
    return static_cast<int>(hipGetLastError());
}
