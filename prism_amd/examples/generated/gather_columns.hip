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
