__device__ void multiply_slot(int __block_id, int __thread_id, char* __smem, float* acc, const __bf16* slot) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0;
        int __thread_id_1 = __thread_id_0 % 256;
        int wave = (__thread_id_1 / 64);
        int row0 = (64 * (wave / 2));
        int col0 = (128 * (wave % 2));
        {
            int __block_id_2 = __block_id_1;
            int __thread_id_2 = __thread_id_1 % 64;
            int lane = __thread_id_2;
            int r = (lane % 16);
            float4 a[4];
            for (int kk = 0; kk < 2; kk++) {
                int k8 = (8 * (((4 * kk) + (lane / 16)) ^ ((r / 2) % 8)));
                for (int i = 0; i < 4; i++) {
                    a[i] = reinterpret_cast<const float4 *>(&slot[((((row0 + (16 * i)) + r) * 64) + k8)])[0];
                }
                for (int j = 0; j < 8; j++) {
                    float4 b = reinterpret_cast<const float4 *>(&slot[((8192 + (((col0 + (16 * j)) + r) * 64)) + k8)])[0];
                    for (int i = 0; i < 4; i++) {
                        {
                            typedef float __acc_t __attribute__((ext_vector_type(4)));
                            __acc_t __acc = {acc[(((8 * i) + j) * 4)], acc[((((8 * i) + j) * 4) + 1)], acc[((((8 * i) + j) * 4) + 2)], acc[((((8 * i) + j) * 4) + 3)]};
                            typedef __bf16 __packet_t __attribute__((ext_vector_type(8)));
                            __acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(__packet_t, a[i]), __builtin_bit_cast(__packet_t, b), __acc, 0, 0, 0);
                            acc[(((8 * i) + j) * 4)] = __acc[0];
                            acc[((((8 * i) + j) * 4) + 1)] = __acc[1];
                            acc[((((8 * i) + j) * 4) + 2)] = __acc[2];
                            acc[((((8 * i) + j) * 4) + 3)] = __acc[3];
                        }
                    }
                }
            }
        }
    }
    return;
}
