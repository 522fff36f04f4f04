__device__ void fill_slot_f32(int __block_id, int __thread_id, char* __smem, float* slot, const float* A_from, const float* B_from, int N, int K, int k_at) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0;
        int __thread_id_1 = __thread_id_0 % 256;
        int w = (__thread_id_1 / 64);
        {
            int __block_id_2 = __block_id_1;
            int __thread_id_2 = __thread_id_1 % 64;
            int lane = __thread_id_2;
            for (int part = 0; part < 4; part++) {
                int arow = ((8 * ((4 * part) + w)) + (lane / 8));
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(&A_from[(((arow * K) + k_at) + (4 * ((lane % 8) ^ ((arow / 2) % 8))))]), (__attribute__((address_space(3))) void*)(&slot[(256 * ((4 * part) + w))]), 16, 0, 0);
            }
            for (int part = 0; part < 8; part++) {
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(&B_from[((((k_at + (4 * part)) + w) * N) + (4 * lane))]), (__attribute__((address_space(3))) void*)(&slot[(4096 + (256 * ((4 * part) + w)))]), 16, 0, 0);
            }
        }
    }
    return;
}
