template<int BM, int BN, int BK, int TM, int TN>
__device__ void multiply_tiles(int __block_id, int __thread_id, char* __smem, float* acc, const float* a_tile, const float* b_tile, int out_r, int out_c) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0 % 1;
        int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
        {
            int __block_id_2 = __block_id_1;
            int __thread_id_2 = __thread_id_1 % 1;
            for (int kk = 0; kk < BK; kk++) {
                for (int i = 0; i < TM; i++) {
                    for (int j = 0; j < TN; j++) {
                        acc[((i * TN) + j)] += (a_tile[(((kk * BM) + (out_r * TM)) + i)] * b_tile[(((kk * BN) + (out_c * TN)) + j)]);
                    }
                }
            }
        }
    }
    return;
}
