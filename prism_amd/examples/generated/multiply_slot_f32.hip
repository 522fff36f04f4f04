__device__ void multiply_slot_f32(int __block_id, int __thread_id, char* __smem, float* acc, const float* slot) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0;
        int __thread_id_1 = __thread_id_0 % 512;
        int wave = (__thread_id_1 / 64);
        int row0 = (64 * (wave / 4));
        int col0 = (64 * (wave % 4));
        {
            int __block_id_2 = __block_id_1;
            int __thread_id_2 = __thread_id_1 % 64;
            int lane = __thread_id_2;
            int l32 = (lane % 32);
            float a[2];
            float b[2];
            for (int kk = 0; kk < 32; kk += 2) {
                int k = (kk + (lane / 32));
                for (int i = 0; i < 2; i++) {
                    a[i] = slot[(((((row0 + (32 * i)) + l32) * 32) + (4 * ((k / 4) ^ ((l32 / 2) % 8)))) + (k % 4))];
                }
                for (int j = 0; j < 2; j++) {
                    b[j] = slot[((((4096 + (k * 256)) + col0) + (32 * j)) + l32)];
                }
                for (int i = 0; i < 2; i++) {
                    for (int j = 0; j < 2; j++) {
                        {
                            typedef float __acc_t __attribute__((ext_vector_type(16)));
                            __acc_t __acc = {acc[((((2 * i) + j) * 16) + 0)], acc[((((2 * i) + j) * 16) + 1)], acc[((((2 * i) + j) * 16) + 2)], acc[((((2 * i) + j) * 16) + 3)], acc[((((2 * i) + j) * 16) + 4)], acc[((((2 * i) + j) * 16) + 5)], acc[((((2 * i) + j) * 16) + 6)], acc[((((2 * i) + j) * 16) + 7)], acc[((((2 * i) + j) * 16) + 8)], acc[((((2 * i) + j) * 16) + 9)], acc[((((2 * i) + j) * 16) + 10)], acc[((((2 * i) + j) * 16) + 11)], acc[((((2 * i) + j) * 16) + 12)], acc[((((2 * i) + j) * 16) + 13)], acc[((((2 * i) + j) * 16) + 14)], acc[((((2 * i) + j) * 16) + 15)]};
                            __acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[j], __acc, 0, 0, 0);
                            acc[((((2 * i) + j) * 16) + 0)] = __acc[0];
                            acc[((((2 * i) + j) * 16) + 1)] = __acc[1];
                            acc[((((2 * i) + j) * 16) + 2)] = __acc[2];
                            acc[((((2 * i) + j) * 16) + 3)] = __acc[3];
                            acc[((((2 * i) + j) * 16) + 4)] = __acc[4];
                            acc[((((2 * i) + j) * 16) + 5)] = __acc[5];
                            acc[((((2 * i) + j) * 16) + 6)] = __acc[6];
                            acc[((((2 * i) + j) * 16) + 7)] = __acc[7];
                            acc[((((2 * i) + j) * 16) + 8)] = __acc[8];
                            acc[((((2 * i) + j) * 16) + 9)] = __acc[9];
                            acc[((((2 * i) + j) * 16) + 10)] = __acc[10];
                            acc[((((2 * i) + j) * 16) + 11)] = __acc[11];
                            acc[((((2 * i) + j) * 16) + 12)] = __acc[12];
                            acc[((((2 * i) + j) * 16) + 13)] = __acc[13];
                            acc[((((2 * i) + j) * 16) + 14)] = __acc[14];
                            acc[((((2 * i) + j) * 16) + 15)] = __acc[15];
                        }
                    }
                }
            }
        }
    }
    return;
}
