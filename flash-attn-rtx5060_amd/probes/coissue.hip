// Hardware probe: how many vector instructions fit next to one v_mfma_f32_32x32x16_f16 before the matrix
// pipe starves, for one and two waves per SIMD (wall-clock throughput on all-zero operands, so that the clock
// stays at its maximum; the counter ticks per instruction are printed as well)
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
#define CK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("HIP error %s line %d\n", hipGetErrorString(e), __LINE__); exit(1);} }while(0)
template <int K, int KIND>
__global__ void __launch_bounds__(512, 1) k(float *out, long long *cyc, int iters, int slot)
{
    f16x8 a, b;
    for (int i = 0; i < 8; ++i) { a[i] = (_Float16)0.0f; b[i] = (_Float16)0.0f; }
    f32x16 acc[4];
    for (int i = 0; i < 4; ++i) for (int r = 0; r < 16; ++r) acc[i][r] = 0.0f;
    float t[8];
    for (int i = 0; i < 8; ++i) t[i] = -0.001f * (float)(threadIdx.x + i);
    const long long t0 = __builtin_amdgcn_s_memtime();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            acc[j & 3] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, acc[j & 3], 0, 0, 0);
#pragma unroll
            for (int v = 0; v < K; ++v) {
                float &x = t[(j * K + v) & 7];
                if (KIND == 0) x = __builtin_fmaf(x, 0.999f, -0.001f);
                if (KIND == 1) x = __builtin_amdgcn_exp2f(x);
                if (KIND == 2) { typedef short s4 __attribute__((ext_vector_type(2))); x = __builtin_amdgcn_fdot2(__builtin_bit_cast(__attribute__((ext_vector_type(2))) _Float16, x), __builtin_bit_cast(__attribute__((ext_vector_type(2))) _Float16, 0x3c003c00), x, false); }
                asm volatile("" : "+v"(x));
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    const long long t1 = __builtin_amdgcn_s_memtime();
    float s = 0;
    for (int i = 0; i < 4; ++i) for (int r = 0; r < 16; ++r) s += acc[i][r];
    for (int i = 0; i < 8; ++i) s += t[i];
    out[blockIdx.x * blockDim.x + threadIdx.x] = s;
    if (threadIdx.x == 0 && blockIdx.x == 0) cyc[slot] = t1 - t0;
}
int main()
{
    float *out; long long *cyc; CK(hipMalloc(&out, 256 * 512 * 4)); CK(hipMalloc(&cyc, 1024)); CK(hipMemset(cyc, 0, 1024));
    const int iters = 500;
    for (int waves = 4; waves <= 8; waves += 4) {
        const int block = waves * 64;
#define RUN(K, KIND, SLOT) hipLaunchKernelGGL((k<K, KIND>), dim3(256), dim3(block), 0, 0, out, cyc, iters, SLOT)
        for (int rep = 0; rep < 2; ++rep) {
            RUN(0, 0, 0); RUN(1, 0, 1); RUN(2, 0, 2); RUN(3, 0, 3); RUN(4, 0, 4); RUN(5, 0, 5); RUN(6, 0, 6); RUN(7, 0, 7); RUN(8, 0, 8); RUN(10, 0, 9);
            RUN(1, 1, 10); RUN(2, 1, 11); RUN(3, 1, 12); RUN(4, 1, 13);
            RUN(1, 2, 14); RUN(2, 2, 15); RUN(4, 2, 16); RUN(6, 2, 17);
            CK(hipDeviceSynchronize());
        }
        {
            hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
            CK(hipEventRecord(e0)); for (int r = 0; r < 50; ++r) RUN(0, 0, 0); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
            float ms; CK(hipEventElapsedTime(&ms, e0, e1));
            const double mf = 50.0 * 256 * waves * iters * 16.0;
            printf("%d waves per block: %.1f TFLOP/s by wall clock (MFMA only, zero data)\n", waves, mf * 32768.0 / ms / 1e9);
            CK(hipEventRecord(e0)); for (int r = 0; r < 50; ++r) RUN(4, 0, 4); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
            CK(hipEventElapsedTime(&ms, e0, e1));
            printf("%d waves per block: %.1f TFLOP/s by wall clock (MFMA + 4 fma)\n", waves, mf * 32768.0 / ms / 1e9);
            CK(hipEventRecord(e0)); for (int r = 0; r < 50; ++r) RUN(7, 0, 7); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
            CK(hipEventElapsedTime(&ms, e0, e1));
            printf("%d waves per block: %.1f TFLOP/s by wall clock (MFMA + 7 fma)\n", waves, mf * 32768.0 / ms / 1e9);
        }
        long long h[32]; CK(hipMemcpy(h, cyc, 256, hipMemcpyDeviceToHost));
        const char *names[18] = {"0 VALU", "1 fma", "2 fma", "3 fma", "4 fma", "5 fma", "6 fma", "7 fma", "8 fma", "10 fma", "1 exp", "2 exp", "3 exp", "4 exp", "1 dot2", "2 dot2", "4 dot2", "6 dot2"};
        for (int i = 0; i < 18; ++i)
            printf("%d wave(s) per SIMD, MFMA + %-7s: %.1f counter ticks per MFMA per wave\n", waves / 4, names[i], (double)h[i] / (iters * 16.0));
    }
    return 0;
}
