__global__ void lookback_scan_by_parts(const uint32_t* x, uint32_t* y, uint32_t* counter, uint64_t* status, int spin_limit) {
    extern __shared__ __align__(128) char __smem[];
    int __block_id_0 = blockIdx.x;
    int __thread_id_0 = __block_id_0 * blockDim.x + threadIdx.x;
    uint32_t tile = take_ticket(__block_id_0, __thread_id_0, __smem, counter);
    {
        const uint32_t* x_tile = x + ((tile * 1024));
        {
            uint32_t* y_tile = y + ((tile * 1024));
            {
                uint64_t* status_blk = status + (0);
                {
                    int __block_id_1 = __block_id_0 % 1;
                    int __thread_id_1 = __block_id_1 * blockDim.x + threadIdx.x;
                    __shared__ uint32_t scanned[1024];
                    scan_rows(__block_id_1, __thread_id_1, __smem, x_tile, scanned);
                    __shared__ uint32_t ends[16];
                    __shared__ uint32_t spare[16];
                    __syncthreads();
                    collect_row_ends(__block_id_1, __thread_id_1, __smem, scanned, ends);
                    __syncthreads();
                    uint32_t* upto = scan_row_ends(__block_id_1, __thread_id_1, __smem, ends, spare);
                    uint32_t total = upto[15];
                    publish(__block_id_1, __thread_id_1, __smem, status_blk, tile, 1, total);
                    uint32_t before = look_back(__block_id_1, __thread_id_1, __smem, status_blk, tile, spin_limit);
                    publish(__block_id_1, __thread_id_1, __smem, status_blk, tile, 2, (before + total));
                    write_back(__block_id_1, __thread_id_1, __smem, y_tile, scanned, upto, before);
                }
            }
        }
    }
}
