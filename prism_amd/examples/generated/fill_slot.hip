__device__ void fill_slot(int __block_id, int __thread_id, char* __smem, __bf16* slot, const __bf16* P_from, const __bf16* Q_from, int K, int k_at) {
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
                int prow = ((8 * ((4 * part) + w)) + (lane / 8));
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(&P_from[(((prow * K) + k_at) + (8 * ((lane % 8) ^ ((prow / 2) % 8))))]), (__attribute__((address_space(3))) void*)(&slot[(512 * ((4 * part) + w))]), 16, 0, 0);
            }
            for (int part = 0; part < 8; part++) {
                int qrow = ((8 * ((4 * part) + w)) + (lane / 8));
                __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(&Q_from[(((qrow * K) + k_at) + (8 * ((lane % 8) ^ ((qrow / 2) % 8))))]), (__attribute__((address_space(3))) void*)(&slot[(8192 + (512 * ((4 * part) + w)))]), 16, 0, 0);
            }
        }
    }
    return;
}
