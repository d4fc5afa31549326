// Hardware probe: issue rates of the vector instructions the softmax uses on gfx950, one wave per SIMD
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#define CK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("HIP error %s line %d\n", hipGetErrorString(e), __LINE__); exit(1);} }while(0)
template <int OP>
__global__ void __launch_bounds__(256, 1) k(float *out, long long *cyc, int iters)
{
    float x[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) x[i] = -0.001f * (float)(threadIdx.x + i);
    const long long t0 = __builtin_readcyclecounter();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            if (OP == 0) x[i] = __builtin_amdgcn_exp2f(x[i]);
            if (OP == 1) x[i] = __builtin_fmaf(x[i], 0.999f, -0.001f);
            if (OP == 2) x[i] = x[i] + 0.001f;
            if (OP == 3) x[i] = __builtin_fmaxf(__builtin_fmaxf(x[i], x[(i + 1) & 15]), x[(i + 2) & 15]);
            if (OP == 4) { typedef _Float16 h2 __attribute__((ext_vector_type(2))); typedef float f2 __attribute__((ext_vector_type(2)));
                           f2 v = {x[i], x[(i + 1) & 15]}; h2 h = __builtin_convertvector(v, h2); x[i] = __builtin_bit_cast(float, h); }
            if (OP == 5) x[i] = __builtin_amdgcn_rcpf(x[i]);
            if (OP == 6) { x[i] = __builtin_fmaf(x[i], 0.999f, -0.001f); if (i % 4 == 0) x[i] = __builtin_amdgcn_exp2f(x[i]); }
        }
    }
    const long long t1 = __builtin_readcyclecounter();
    float s = 0;
#pragma unroll
    for (int i = 0; i < 16; ++i) s += x[i];
    out[blockIdx.x * blockDim.x + threadIdx.x] = s;
    if (threadIdx.x == 0 && blockIdx.x == 0) cyc[OP] = t1 - t0;
}
int main()
{
    float *out; long long *cyc; CK(hipMalloc(&out, 256 * 256 * 4)); CK(hipMalloc(&cyc, 64)); CK(hipMemset(cyc, 0, 64));
    const int iters = 2000;
    const char *names[7] = {"v_exp_f32", "v_fma_f32", "v_add_f32", "v_max3_f32", "v_cvt_pk_f16_f32", "v_rcp_f32", "3 fma : 1 exp mix"};
    for (int rep = 0; rep < 2; ++rep) {
        hipLaunchKernelGGL(k<0>, dim3(256), dim3(256), 0, 0, out, cyc, iters);
        hipLaunchKernelGGL(k<1>, dim3(256), dim3(256), 0, 0, out, cyc, iters);
        hipLaunchKernelGGL(k<2>, dim3(256), dim3(256), 0, 0, out, cyc, iters);
        hipLaunchKernelGGL(k<3>, dim3(256), dim3(256), 0, 0, out, cyc, iters);
        hipLaunchKernelGGL(k<4>, dim3(256), dim3(256), 0, 0, out, cyc, iters);
        hipLaunchKernelGGL(k<5>, dim3(256), dim3(256), 0, 0, out, cyc, iters);
        hipLaunchKernelGGL(k<6>, dim3(256), dim3(256), 0, 0, out, cyc, iters);
        CK(hipDeviceSynchronize());
    }
    long long h[8]; CK(hipMemcpy(h, cyc, 64, hipMemcpyDeviceToHost));
    // s_memtime / readcyclecounter ticks at the 100 MHz reference on this chip? print raw per-instruction ticks and a timed run
    for (int i = 0; i < 7; ++i) printf("%-22s %.3f counter ticks per instruction (one wave per SIMD)\n", names[i], (double)h[i] / (iters * 64.0));
    hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    auto timed = [&](auto kern, const char *name) {
        CK(hipEventRecord(e0)); for (int r = 0; r < 20; ++r) hipLaunchKernelGGL(kern, dim3(256), dim3(256), 0, 0, out, cyc, iters); CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
        float ms; CK(hipEventElapsedTime(&ms, e0, e1));
        printf("%-22s %.2f ns per wave instruction (wall clock; 4 cycles at 2.4 GHz = 1.67 ns)\n", name, ms * 1e6 / 20.0 / (iters * 64.0));
    };
    timed(k<0>, names[0]); timed(k<1>, names[1]); timed(k<2>, names[2]); timed(k<3>, names[3]); timed(k<4>, names[4]); timed(k<5>, names[5]); timed(k<6>, names[6]);
    return 0;
}
