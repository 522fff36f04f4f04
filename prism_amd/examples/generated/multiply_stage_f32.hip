__device__ void multiply_stage_f32(int __block_id, int __thread_id, char* __smem, float* acc, const float* stage) {
    int __block_id_0 = __block_id;
    int __thread_id_0 = __thread_id;
    {
        int __block_id_1 = __block_id_0;
        int __thread_id_1 = __thread_id_0 % 1024;
        int wave = (__thread_id_1 / 64);
        int row0 = (32 * (wave / 2));
        int col0 = (128 * (wave % 2));
        {
            int __block_id_2 = __block_id_1;
            int __thread_id_2 = __thread_id_1 % 64;
            int lane = __thread_id_2;
            int l32 = (lane % 32);
            int half = (lane / 32);
            float a[4];
            float b[16];
            for (int s = 0; s < 4; s++) {
                reinterpret_cast<float4 *>(&a[0])[0] = reinterpret_cast<const float4 *>(&stage[(((row0 + l32) * 32) + (4 * (((2 * s) + half) ^ ((l32 / 2) % 8))))])[0];
                for (int jj = 0; jj < 4; jj++) {
                    reinterpret_cast<float4 *>(&b[(4 * jj)])[0] = reinterpret_cast<const float4 *>(&stage[(((8192 + ((((8 * s) + (4 * half)) + jj) * 256)) + col0) + (4 * l32))])[0];
                }
                for (int jj = 0; jj < 4; jj++) {
                    for (int j = 0; j < 4; j++) {
                        {
                            typedef float __acc_t __attribute__((ext_vector_type(16)));
                            __acc_t __acc = {acc[((j * 16) + 0)], acc[((j * 16) + 1)], acc[((j * 16) + 2)], acc[((j * 16) + 3)], acc[((j * 16) + 4)], acc[((j * 16) + 5)], acc[((j * 16) + 6)], acc[((j * 16) + 7)], acc[((j * 16) + 8)], acc[((j * 16) + 9)], acc[((j * 16) + 10)], acc[((j * 16) + 11)], acc[((j * 16) + 12)], acc[((j * 16) + 13)], acc[((j * 16) + 14)], acc[((j * 16) + 15)]};
                            __acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a[jj], b[((4 * jj) + j)], __acc, 0, 0, 0);
                            acc[((j * 16) + 0)] = __acc[0];
                            acc[((j * 16) + 1)] = __acc[1];
                            acc[((j * 16) + 2)] = __acc[2];
                            acc[((j * 16) + 3)] = __acc[3];
                            acc[((j * 16) + 4)] = __acc[4];
                            acc[((j * 16) + 5)] = __acc[5];
                            acc[((j * 16) + 6)] = __acc[6];
                            acc[((j * 16) + 7)] = __acc[7];
                            acc[((j * 16) + 8)] = __acc[8];
                            acc[((j * 16) + 9)] = __acc[9];
                            acc[((j * 16) + 10)] = __acc[10];
                            acc[((j * 16) + 11)] = __acc[11];
                            acc[((j * 16) + 12)] = __acc[12];
                            acc[((j * 16) + 13)] = __acc[13];
                            acc[((j * 16) + 14)] = __acc[14];
                            acc[((j * 16) + 15)] = __acc[15];
                        }
                    }
                }
            }
        }
    }
    return;
}
