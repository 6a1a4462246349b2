// mfma_rate.hip -- what the matrix pipes sustain with one wave per SIMD issuing nothing but
// v_mfma_f32_16x16x32_f16 on independent accumulator tiles: per grid size (one workgroup of 4
// waves per CU), for accumulators in VGPRs and in AGPRs, on random and on all-zero operands
// (the clocks this GPU holds depend on the data: more toggling bits, more power, lower clock).
//
//   build: hipcc --offload-arch=gfx950 -O3 -o mfma_rate mfma_rate.hip
//   run:   ./mfma_rate
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
#define CK(x)                                                                          \
    do {                                                                               \
        hipError_t e_ = (x);                                                           \
        if (e_ != hipSuccess) {                                                        \
            printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);      \
            exit(1);                                                                   \
        }                                                                              \
    } while (0)

// NT independent accumulator tiles per wave; the operands never change
template <int NT, bool AGPR>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void rate(float *out, int iters, int random)
{
    half8_t a, b;
    unsigned s = threadIdx.x * 2654435761u + blockIdx.x * 40503u + 12345u;
    for (int i = 0; i < 8; ++i) {
        s = s * 1664525u + 1013904223u;
        a[i] = random ? (_Float16)(((s >> 8) & 0xFFFF) / 32768.0f - 1.0f) : (_Float16)0.0f;
        s = s * 1664525u + 1013904223u;
        b[i] = random ? (_Float16)(((s >> 8) & 0xFFFF) / 32768.0f - 1.0f) : (_Float16)0.0f;
    }
    float4_t acc[NT];
#pragma unroll
    for (int i = 0; i < NT; ++i) acc[i] = float4_t{0, 0, 0, 0};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < NT; ++i) {
            if constexpr (AGPR) asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(acc[i]) : "v"(a), "v"(b));
            else asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(acc[i]) : "v"(a), "v"(b));
        }
    }
    float4_t sum = float4_t{0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < NT; ++i) sum += acc[i];
    if (sum[0] == 12345.678f) out[threadIdx.x] = sum[1] + sum[2] + sum[3];
}

template <int NT, bool AGPR>
void run(const char *name, int grid, float *d, int random)
{
    const int iters = 4096 / NT * 16;   // 65536 MFMAs per wave
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    hipLaunchKernelGGL((rate<NT, AGPR>), dim3(grid), dim3(256), 0, 0, d, iters, random);
    CK(hipEventRecord(e0, 0));
    for (int r = 0; r < 5; ++r) hipLaunchKernelGGL((rate<NT, AGPR>), dim3(grid), dim3(256), 0, 0, d, iters, random);
    CK(hipEventRecord(e1, 0));
    CK(hipEventSynchronize(e1));
    float ms;
    CK(hipEventElapsedTime(&ms, e0, e1));
    const double us = ms * 1000 / 5;
    const double mfmas = (double)iters * NT;   // per wave
    const double flops = mfmas * 16384.0 * 4 * grid;
    printf("%-22s %-7s %4d CUs: %8.1f us, %5.2f ns per MFMA per SIMD, %6.0f TFLOP/s\n", name, random ? "random" : "zeros",
           grid, us, us * 1000 / mfmas, flops / us * 1e-6);
}

int main()
{
    float *d;
    CK(hipMalloc(&d, 4096));
    for (int random = 1; random >= 0; --random)
        for (int grid : {256, 32, 1}) {
            run<16, false>("16 tiles in VGPRs", grid, d, random);
            run<64, true>("64 tiles in AGPRs", grid, d, random);
        }
    return 0;
}
