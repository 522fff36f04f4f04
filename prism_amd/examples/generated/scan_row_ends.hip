__device__ uint32_t* scan_row_ends(int __block_id, int __thread_id, char* __smem, uint32_t* ends, uint32_t* spare) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0 % 1;
        int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
        uint32_t t = __thread_id_1;
        uint32_t stride = 1;
        while ((stride < 16)) {
            {
                uint32_t* end_one = ends + (t);
                {
                    uint32_t* spare_one = spare + (t);
                    {
                        int __block_id_2 = __block_id_1;
                        int __thread_id_2 = __thread_id_1 % 1;
                        if ((t < 16)) {
                            if ((t >= stride)) {
                                spare_one[0] = (ends[t] + ends[(t - stride)]);
                            } else {
                                spare_one[0] = ends[t];
                            }
                        }
                        __syncthreads();
                        if ((t < 16)) {
                            end_one[0] = spare[t];
                        }
                    }
                }
            }
            stride *= 2;
            __syncthreads();
        }
    }
    return ends;
}
