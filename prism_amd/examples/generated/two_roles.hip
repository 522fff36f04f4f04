__global__ void two_roles(const int* x, int* y, int n) {
    extern __shared__ __align__(128) char __smem[];
    int __block_id_0 = blockIdx.x;
    int __thread_id_0 = __block_id_0 * blockDim.x + threadIdx.x;
    int base = (__block_id_0 * 256);
    {
        int* y_mine = y + (base);
        {
            int __block_id_1 = __block_id_0 % 1;
            int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
            {
                int __block_id_2 = __block_id_1;
                int __thread_id_2 = __thread_id_1;
                if (__thread_id_2 >= 0 && __thread_id_2 < 128) {
                    int t = __thread_id_2;
                    {
                        int __block_id_3 = __block_id_2;
                        int __thread_id_3 = __thread_id_2 % 1;
                        if (((base + t) < n)) {
                            y_mine[t] = (x[(base + t)] * 2);
                        }
                    }
                }
            }
            {
                int __block_id_2 = __block_id_1;
                int __thread_id_2 = __thread_id_1 - 128;
                if (__thread_id_2 >= 0 && __thread_id_2 < 128) {
                    int t = __thread_id_2;
                    {
                        int __block_id_3 = __block_id_2;
                        int __thread_id_3 = __thread_id_2 % 1;
                        if ((((base + 128) + t) < n)) {
                            y_mine[(128 + t)] = (x[((base + 128) + t)] + 1);
                        }
                    }
                }
            }
        }
    }
}
