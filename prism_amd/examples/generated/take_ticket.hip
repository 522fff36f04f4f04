__device__ uint32_t take_ticket(int __block_id, int __thread_id, char* __smem, uint32_t* counter) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    __shared__ uint32_t ticket;
    if (threadIdx.x == 0) ticket = atomicAdd(counter, 1u);
    __syncthreads();
    return ticket;
}
