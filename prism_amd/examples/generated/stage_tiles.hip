template<int BM, int BN, int BK, int THREADS>
__device__ void stage_tiles(int __block_id, int __thread_id, char* __smem, int N, int K, const float* A_from, const float* B_from, float* a_tile, float* b_tile) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0 % 1;
        int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
        const int t = __thread_id_1;
        {
            float* a_mine = a_tile + (0);
            {
                float* b_mine = b_tile + (0);
                {
                    int __block_id_2 = __block_id_1;
                    int __thread_id_2 = __thread_id_1 % 1;
                    for (int e = t; e < (BM * BK); e += THREADS) {
                        a_mine[(((e % BK) * BM) + (e / BK))] = A_from[(((e / BK) * K) + (e % BK))];
                    }
                    for (int e = t; e < (BK * BN); e += THREADS) {
                        b_mine[e] = B_from[(((e / BN) * N) + (e % BN))];
                    }
                }
            }
        }
    }
    return;
}
