// Hardware probe: what the matrix cores sustain under the chip's power management, by operand data, accumulator
// order and the instructions issued next to them (LDS reads, vector ALU work), with socket power and XCD clocks
// sampled from amd-smi while the loop runs.  Bounds what any attention kernel can reach on this part.
// Usage: mfma_power <variant> <seconds>;  variant = mode + 10 * data (data 0: N(0, 0.25^2), 1: zeros, 2: probabilities)
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <cmath>
#include <thread>
#include <atomic>
#include <string>
#include <vector>
#include <chrono>
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
#define CK(x) do{hipError_t e=(x); if(e!=hipSuccess){printf("HIP error %s line %d\n", hipGetErrorString(e), __LINE__); exit(1);} }while(0)

// MODE 0: 8 accumulators round-robin, 8 A and 8 B fragments rotating (each MFMA different operands)
// MODE 1: chains of 8 MFMAs into one accumulator, then the next accumulator
// MODE 2: like 0 but bf16
// MODE 3 / 4: MODE 0 with idle cycles after every MFMA (matrix pipe about 80 % / 55 % busy)
// MODE 5 / 6: MODE 0 with the A operand of every MFMA / every second MFMA freshly read from LDS (ds_read_b128)
// MODE 7: MODE 0 with four vector instructions (fma, exp2, add, max) per MFMA
// MODE 8: 5 and 7 together
// MODE 9: 5 with the vector instructions of 7 on every second MFMA only
template <int MODE>
__global__ void __launch_bounds__(512, 1) k(const uint4 *a_src, const uint4 *b_src, float *out, int iters)
{
    const int lane = threadIdx.x & 63;
    __shared__ uint4 lds[4096];     // 64 KiB
    if (MODE == 5 || MODE == 6 || MODE == 8 || MODE == 9) {
        for (int i = threadIdx.x; i < 4096; i += blockDim.x) lds[i] = a_src[i & 511];
        __syncthreads();
    }
    float t[8], l[2] = {0.0f, 0.0f}, mx = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i) t[i] = -0.01f * (float)(lane + i);
    uint4 af[8], bf[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) { af[i] = a_src[(i * 64 + lane)]; bf[i] = b_src[(i * 64 + lane)]; }
    f32x16 acc[8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = 0.0f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int j = 0; j < 64; ++j) {
            // the fragment read here is used four MFMAs later (the ring of eight is otherwise stationary)
            if (MODE == 5 || MODE == 8 || MODE == 9 || ((MODE == 6) && (j & 1) == 0))
                af[(j + 4) & 7] = lds[((threadIdx.x >> 6) * 512 + ((j * 64 + lane) & 511)) & 4095];
            const int ai = MODE == 1 ? (j & 7) : (j & 7), bi = MODE == 1 ? ((j >> 3) & 7) : ((j + (j >> 3)) & 7);
            const int ci = MODE == 1 ? (j >> 3) : (j & 7);
            if (MODE == 2)
                acc[ci] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, af[ai]), __builtin_bit_cast(bf16x8, bf[bi]), acc[ci], 0, 0, 0);
            else
                acc[ci] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, af[ai]), __builtin_bit_cast(f16x8, bf[bi]), acc[ci], 0, 0, 0);
            if (MODE == 3) asm volatile("s_nop 7");
            if (MODE == 4) asm volatile("s_nop 15\n\ts_nop 9");
            if (MODE == 7 || MODE == 8 || (MODE == 9 && (j & 1) == 0)) {
                t[j & 7] = __builtin_fmaf(t[j & 7], 0.999f, -0.001f);
                const float e = __builtin_amdgcn_exp2f(t[j & 7]);
                l[j & 1] += e;
                mx = fmaxf(mx, e);
                asm volatile("" : "+v"(l[j & 1]), "+v"(mx));
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // keep magnitudes bounded without changing the instruction mix much: one cheap op per accumulator
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i][0] *= 0.5f;
    }
    float s = l[0] + l[1] + mx;
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) s += acc[i][r];
    out[blockIdx.x * blockDim.x + threadIdx.x] = s;
}

static std::string smi()
{
    std::string r; char buf[512];
    FILE *f = popen("amd-smi metric --power --clock 2>&1 | grep -E 'SOCKET_POWER|GFX_[0-7]:|^ +CLK:' | head -20 | tr '\\n' ' '", "r");
    if (!f) return "popen failed";
    while (fgets(buf, sizeof buf, f)) r += buf;
    pclose(f);
    return r;
}

int main(int argc, char **argv)
{
    const int variant = argc > 1 ? atoi(argv[1]) : 0;      // mode + 10 * data (0 normal, 1 zero, 2 uniform 0..1 "P-like")
    const double seconds = argc > 2 ? atof(argv[2]) : 4.0;
    const int mode = variant % 10, data = variant / 10;
    std::vector<uint16_t> ha(8 * 64 * 8), hb(8 * 64 * 8);
    srand(1);
    auto gauss = []() { double u = (rand() + 1.0) / (RAND_MAX + 2.0), v = (rand() + 1.0) / (RAND_MAX + 2.0); return sqrt(-2 * log(u)) * cos(6.283185307 * v); };
    for (size_t i = 0; i < ha.size(); ++i) {
        float x = data == 1 ? 0.0f : (float)gauss() * 0.25f, y = data == 1 ? 0.0f : data == 2 ? (float)exp2(-8.0 * rand() / RAND_MAX) * 0.05f : (float)gauss() * 0.25f;
        if (mode == 2) { __bf16 p = (__bf16)x, q = (__bf16)y; memcpy(&ha[i], &p, 2); memcpy(&hb[i], &q, 2); }
        else { _Float16 p = (_Float16)x, q = (_Float16)y; memcpy(&ha[i], &p, 2); memcpy(&hb[i], &q, 2); }
    }
    uint4 *da, *db; float *dout;
    const int grid = 512, block = 512, iters = 2000;
    CK(hipMalloc(&da, ha.size() * 2)); CK(hipMalloc(&db, hb.size() * 2)); CK(hipMalloc(&dout, grid * block * 4));
    CK(hipMemcpy(da, ha.data(), ha.size() * 2, hipMemcpyHostToDevice)); CK(hipMemcpy(db, hb.data(), hb.size() * 2, hipMemcpyHostToDevice));
    auto launch = [&]() {
        switch (mode) {
        case 0: hipLaunchKernelGGL(k<0>, dim3(grid), dim3(block), 0, 0, da, db, dout, iters); break;
        case 1: hipLaunchKernelGGL(k<1>, dim3(grid), dim3(block), 0, 0, da, db, dout, iters); break;
        case 2: hipLaunchKernelGGL(k<2>, dim3(grid), dim3(block), 0, 0, da, db, dout, iters); break;
        case 3: hipLaunchKernelGGL(k<3>, dim3(grid), dim3(block), 0, 0, da, db, dout, iters); break;
        case 4: hipLaunchKernelGGL(k<4>, dim3(grid), dim3(block), 0, 0, da, db, dout, iters); break;
        case 5: hipLaunchKernelGGL(k<5>, dim3(grid), dim3(block), 0, 0, da, db, dout, iters); break;
        case 6: hipLaunchKernelGGL(k<6>, dim3(grid), dim3(block), 0, 0, da, db, dout, iters); break;
        case 7: hipLaunchKernelGGL(k<7>, dim3(grid), dim3(block), 0, 0, da, db, dout, iters); break;
        case 8: hipLaunchKernelGGL(k<8>, dim3(grid), dim3(block), 0, 0, da, db, dout, iters); break;
        default: hipLaunchKernelGGL(k<9>, dim3(grid), dim3(block), 0, 0, da, db, dout, iters); break;
        }
    };
    launch(); CK(hipDeviceSynchronize());
    hipEvent_t e0, e1; CK(hipEventCreate(&e0)); CK(hipEventCreate(&e1));
    std::atomic<bool> done{false};
    std::string sample;
    std::thread t([&]() { std::this_thread::sleep_for(std::chrono::milliseconds((int)(seconds * 600))); sample = smi(); });
    auto t0 = std::chrono::steady_clock::now();
    int launches = 0;
    CK(hipEventRecord(e0));
    while (std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() < seconds) { for (int i = 0; i < 4; ++i) launch(); launches += 4; CK(hipStreamSynchronize(0)); }
    CK(hipEventRecord(e1)); CK(hipEventSynchronize(e1));
    t.join();
    float ms; CK(hipEventElapsedTime(&ms, e0, e1));
    const double flops = (double)launches * grid * (block / 64) * (double)iters * 64 * 32768.0;
    printf("variant %d (mode %d data %d): %.1f TFLOP/s = %.1f %% of 2516.6 | %s\n", variant, mode, data, flops / ms / 1e9, flops / ms / 1e9 / 25.166, sample.c_str());
    return 0;
}
