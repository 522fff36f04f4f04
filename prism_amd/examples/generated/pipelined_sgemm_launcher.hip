#include <hip/hip_runtime.h>
#include <cstddef>
#include <cstdint>

__device__ void fill_stage_f32(int __block_id, int __thread_id, char* __smem, float* stage, const float* A_from, const float* B_from, int N, int K, int k_at) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0;
        int __thread_id_1 = __thread_id_0 % 1024;
        int w = (__thread_id_1 / 64);
        {
            int __block_id_2 = __block_id_1;
            int __thread_id_2 = __thread_id_1 % 64;
            int lane = __thread_id_2;
            for (int part = 0; part < 2; part++) {
                int arow = ((8 * ((16 * part) + w)) + (lane / 8));
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(&A_from[(((arow * K) + k_at) + (4 * ((lane % 8) ^ ((arow / 2) % 8))))]), (__attribute__((address_space(3))) void*)(&stage[(256 * ((16 * part) + w))]), 16, 0, 0);
            }
            for (int part = 0; part < 2; part++) {
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(&B_from[((((k_at + (16 * part)) + w) * N) + (4 * lane))]), (__attribute__((address_space(3))) void*)(&stage[(8192 + (256 * ((16 * part) + w)))]), 16, 0, 0);
            }
        }
    }
    return;
}

__device__ void multiply_stage_f32(int __block_id, int __thread_id, char* __smem, float* acc, const float* stage) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0;
        int __thread_id_1 = __thread_id_0 % 1024;
        int wave = (__thread_id_1 / 64);
        int row0 = (32 * (wave / 2));
        int col0 = (128 * (wave % 2));
        {
            int __block_id_2 = __block_id_1;
            int __thread_id_2 = __thread_id_1 % 64;
            int lane = __thread_id_2;
            int l32 = (lane % 32);
            int half = (lane / 32);
            float a[4];
            float b[16];
            for (int s = 0; s < 4; s++) {
                reinterpret_cast<float4 *>(&a[0])[0] = reinterpret_cast<const float4 *>(&stage[(((row0 + l32) * 32) + (4 * (((2 * s) + half) ^ ((l32 / 2) % 8))))])[0];
                for (int jj = 0; jj < 4; jj++) {
                    reinterpret_cast<float4 *>(&b[(4 * jj)])[0] = reinterpret_cast<const float4 *>(&stage[(((8192 + ((((8 * s) + (4 * half)) + jj) * 256)) + col0) + (4 * l32))])[0];
                }
                for (int jj = 0; jj < 4; jj++) {
                    for (int j = 0; j < 4; j++) {
                        {
                            typedef float __acc_t __attribute__((ext_vector_type(16)));
                            __acc_t __acc = {acc[((j * 16) + 0)], acc[((j * 16) + 1)], acc[((j * 16) + 2)], acc[((j * 16) + 3)], acc[((j * 16) + 4)], acc[((j * 16) + 5)], acc[((j * 16) + 6)], acc[((j * 16) + 7)], acc[((j * 16) + 8)], acc[((j * 16) + 9)], acc[((j * 16) + 10)], acc[((j * 16) + 11)], acc[((j * 16) + 12)], acc[((j * 16) + 13)], acc[((j * 16) + 14)], acc[((j * 16) + 15)]};
                            __acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[jj], b[((4 * jj) + j)], __acc, 0, 0, 0);
                            acc[((j * 16) + 0)] = __acc[0];
                            acc[((j * 16) + 1)] = __acc[1];
                            acc[((j * 16) + 2)] = __acc[2];
                            acc[((j * 16) + 3)] = __acc[3];
                            acc[((j * 16) + 4)] = __acc[4];
                            acc[((j * 16) + 5)] = __acc[5];
                            acc[((j * 16) + 6)] = __acc[6];
                            acc[((j * 16) + 7)] = __acc[7];
                            acc[((j * 16) + 8)] = __acc[8];
                            acc[((j * 16) + 9)] = __acc[9];
                            acc[((j * 16) + 10)] = __acc[10];
                            acc[((j * 16) + 11)] = __acc[11];
                            acc[((j * 16) + 12)] = __acc[12];
                            acc[((j * 16) + 13)] = __acc[13];
                            acc[((j * 16) + 14)] = __acc[14];
                            acc[((j * 16) + 15)] = __acc[15];
                        }
                    }
                }
            }
        }
    }
    return;
}

__global__ __launch_bounds__(1024) void pipelined_sgemm(int M, int N, int K, float alpha, const float* A, const float* B, float beta, float* C, int tiles_n) {
    extern __shared__ __align__(128) char __smem[];
    int __block_id_0 = blockIdx.x;
    int __thread_id_0 = __block_id_0 * blockDim.x + threadIdx.x;
    const int per_xcd = (((M / 256) * tiles_n) / 8);
    const int t = (((__block_id_0 % 8) * per_xcd) + (__block_id_0 / 8));
    const int tile_r = ((8 * (t / (8 * tiles_n))) + (t % 8));
    const int tile_c = ((t % (8 * tiles_n)) / 8);
    {
        const float* A_rows = A + (((tile_r * 256) * K));
        {
            const float* B_cols = B + ((tile_c * 256));
            {
                float* C_tile = C + ((((tile_r * 256) * N) + (tile_c * 256)));
                {
                    int __block_id_1 = __block_id_0 % 1;
                    int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
                    __shared__ float first[16384];
                    __shared__ float second[16384];
                    float acc[64] = {0};
                    fill_stage_f32(__block_id_1, __thread_id_1, __smem, first, A_rows, B_cols, N, K, 0);
                    __syncthreads();
                    for (int k0 = 0; k0 < K; k0 += 64) {
                        fill_stage_f32(__block_id_1, __thread_id_1, __smem, second, A_rows, B_cols, N, K, (k0 + 32));
                        multiply_stage_f32(__block_id_1, __thread_id_1, __smem, acc, first);
                        __syncthreads();
                        if (((k0 + 64) < K)) {
                            fill_stage_f32(__block_id_1, __thread_id_1, __smem, first, A_rows, B_cols, N, K, (k0 + 64));
                        }
                        multiply_stage_f32(__block_id_1, __thread_id_1, __smem, acc, second);
                        __syncthreads();
                    }
                    {
                        float* C_mine = C_tile + (0);
                        int wave = (__thread_id_1 / 64);
                        {
                            int __block_id_2 = __block_id_1;
                            int __thread_id_2 = __thread_id_1 % 64;
                            int lane = __thread_id_2;
                            {
                                int __block_id_3 = __block_id_2;
                                int __thread_id_3 = __thread_id_2 % 1;
                                for (int v = 0; v < 16; v++) {
                                    for (int j = 0; j < 4; j++) {
                                        int at = ((((((((32 * (wave / 2)) + (8 * (v / 4))) + (4 * (lane / 32))) + (v % 4)) * N) + (128 * (wave % 2))) + (4 * (lane % 32))) + j);
                                        C_mine[at] = ((alpha * acc[((j * 16) + v)]) + (beta * C_mine[at]));
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

extern "C" int pipelined_sgemm_launch(int M, int N, int K, float alpha, const float* A, const float* B, float beta, float* C, int tiles_n, unsigned grid_blocks, void* stream) {
    if (grid_blocks == 0) return 0;
    pipelined_sgemm<<<dim3(grid_blocks), dim3(1024), 0, static_cast<hipStream_t>(stream)>>>(M, N, K, alpha, A, B, beta, C, tiles_n);
    return static_cast<int>(hipGetLastError());
}
