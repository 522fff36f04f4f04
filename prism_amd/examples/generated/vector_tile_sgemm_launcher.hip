#include <hip/hip_runtime.h>
#include <cstddef>
#include <cstdint>

template<int BM, int BN, int BK, int TM, int TN>
__global__ __launch_bounds__((BM * BN) / (TM * TN)) void vector_tile_sgemm(int M, int N, int K, float alpha, float* A, float* B, float beta, float* C, int tiles_n) {
    extern __shared__ __align__(128) char __smem[];
    int __block_id_0 = blockIdx.x;
    int __thread_id_0 = __block_id_0 * blockDim.x + threadIdx.x;
    const int tile_r = (__block_id_0 / tiles_n);
    const int tile_c = (__block_id_0 % tiles_n);
    {
        float* A_rows = A + (((tile_r * BM) * K));
        {
            float* B_cols = B + ((tile_c * BN));
            {
                float* C_tile = C + ((((tile_r * BM) * N) + (tile_c * BN)));
                {
                    int __block_id_1 = __block_id_0 % 1;
                    int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
                    float (&a_lds)[1024] = *((float (*)[1024])(__smem + 0));
                    float (&b_lds)[1024] = *((float (*)[1024])(__smem + 4096));
                    const int t = __thread_id_1;
                    const int out_r = (t / (BN / TN));
                    const int out_c = (t % (BN / TN));
                    const int a_row = (t / (BK / 4));
                    const int a_quad = (t % (BK / 4));
                    const int b_row = (t / (BN / 4));
                    const int b_quad = (t % (BN / 4));
                    float acc[64] = {0};
                    float a_reg[8] = {0};
                    float b_reg[8] = {0};
                    for (int k0 = 0; k0 < K; k0 += BK) {
                        {
                            int __block_id_2 = __block_id_1;
                            int __thread_id_2 = __thread_id_1 % 1;
                            float4 quad = reinterpret_cast<float4 *>(&A_rows[(((a_row * K) + k0) + (a_quad * 4))])[0];
                            a_lds[(((((a_row * BK) + (a_quad * 4)) % BK) * BM) + (((a_row * BK) + (a_quad * 4)) / BK))] = quad.x;
                            a_lds[((((((a_row * BK) + (a_quad * 4)) + 1) % BK) * BM) + ((((a_row * BK) + (a_quad * 4)) + 1) / BK))] = quad.y;
                            a_lds[((((((a_row * BK) + (a_quad * 4)) + 2) % BK) * BM) + ((((a_row * BK) + (a_quad * 4)) + 2) / BK))] = quad.z;
                            a_lds[((((((a_row * BK) + (a_quad * 4)) + 3) % BK) * BM) + ((((a_row * BK) + (a_quad * 4)) + 3) / BK))] = quad.w;
                            reinterpret_cast<float4 *>(&b_lds[((b_row * BN) + (b_quad * 4))])[0] = reinterpret_cast<float4 *>(&B_cols[(((k0 + b_row) * N) + (b_quad * 4))])[0];
                            __syncthreads();
                            for (int kk = 0; kk < BK; kk++) {
                                for (int i = 0; i < TM; i++) {
                                    a_reg[i] = a_lds[(((kk * BM) + (out_r * TM)) + i)];
                                }
                                for (int j = 0; j < TN; j++) {
                                    b_reg[j] = b_lds[(((kk * BN) + (out_c * TN)) + j)];
                                }
                                for (int i = 0; i < TM; i++) {
                                    for (int j = 0; j < TN; j++) {
                                        acc[((i * TN) + j)] += (a_reg[i] * b_reg[j]);
                                    }
                                }
                            }
                        }
                        __syncthreads();
                    }
                    for (int i = 0; i < TM; i++) {
                        for (int j = 0; j < TN; j += 4) {
                            {
                                float* c4 = C_tile + ((((((out_r * TM) + i) * N) + (out_c * TN)) + j));
                                {
                                    int __block_id_2 = __block_id_1;
                                    int __thread_id_2 = __thread_id_1 % 1;
                                    float4 was = reinterpret_cast<float4 *>(&c4[0])[0];
                                    was.x = ((alpha * acc[((i * TN) + j)]) + (beta * was.x));
                                    was.y = ((alpha * acc[(((i * TN) + j) + 1)]) + (beta * was.y));
                                    was.z = ((alpha * acc[(((i * TN) + j) + 2)]) + (beta * was.z));
                                    was.w = ((alpha * acc[(((i * TN) + j) + 3)]) + (beta * was.w));
                                    reinterpret_cast<float4 *>(&c4[0])[0] = was;
                                }
                            }
                        }
                    }
                }
            }
        }
    }
}

extern "C" int vector_tile_sgemm_launch(int M, int N, int K, float alpha, float* A, float* B, float beta, float* C, int tiles_n, unsigned grid_blocks, void* stream) {
    if (grid_blocks == 0) return 0;
    vector_tile_sgemm<128, 128, 8, 8, 8><<<dim3(grid_blocks), dim3(256), 8192, static_cast<hipStream_t>(stream)>>>(M, N, K, alpha, A, B, beta, C, tiles_n);
    return static_cast<int>(hipGetLastError());
}
