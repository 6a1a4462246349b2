// tzgemm_large_probe.hip -- the large-tile tzgemm kernel alone in a plain HIP program: its time
// at a shape, on zero and on random operands, and -- built with TZL_KNOCK_OUT_LOADS,
// TZL_KNOCK_OUT_BARRIER or TZL_KNOCK_OUT_STORES -- what the global->LDS loads and the workgroup
// barrier of the steady K loop and the C stores cost (those builds compute wrong results on
// purpose).
//
//   build: hipcc --offload-arch=gfx950 -O3 -std=c++17 -ffp-contract=off -Xclang -target-feature
//          -Xclang -packed-fp32-ops [-DTZL_KNOCK_OUT_...] -o tzgemm_large_probe tzgemm_large_probe.hip
//   run:   ./tzgemm_large_probe [M N K]        (default 4096 4096 4096)
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../kernels/tzgemm_large.h"

#define CK(x)                                                                          \
    do {                                                                               \
        hipError_t e_ = (x);                                                           \
        if (e_ != hipSuccess) {                                                        \
            printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);      \
            exit(1);                                                                   \
        }                                                                              \
    } while (0)

__global__ __launch_bounds__(TZ_THREADS) __attribute__((amdgpu_waves_per_eu(1, 1))) void probe(
    _Float16 *A, _Float16 *B, float *C, int M, int N, int K)
{
    __shared__ __align__(16) char tz_lds[TZ_LDS_BYTES];
    tk::tzgemm_role_large<8, 8>(A, B, C, M, N, K, (int)blockIdx.x, (int)gridDim.x, 0, (M / 64) * (N / 64),
                                (int)threadIdx.x, tz_lds, (size_t)M * (size_t)N * sizeof(float) > TZ_LARGE_STREAM_C_BYTES);
}

int main(int argc, char **argv)
{
    const int M = argc > 3 ? atoi(argv[1]) : 4096, N = argc > 3 ? atoi(argv[2]) : 4096, K = argc > 3 ? atoi(argv[3]) : 4096;
    if (M % 256 || N % 256 || K % 128 || M <= 0 || N <= 0 || K <= 0) {
        printf("M and N must be multiples of 256, K of 128\n");
        return 1;
    }
    _Float16 *A, *B;
    float *C;
    CK(hipMalloc(&A, (size_t)M * K * 2));
    CK(hipMalloc(&B, (size_t)N * K * 2));
    CK(hipMalloc(&C, (size_t)M * N * 4));
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    const int grid = 256;
    for (int random = 0; random < 2; ++random) {
        std::vector<_Float16> h((size_t)(M > N ? M : N) * K);
        unsigned s = 12345u;
        for (auto &v : h) {
            s = s * 1664525u + 1013904223u;
            v = random ? (_Float16)(((s >> 8) & 0xFFFF) / 32768.0f - 1.0f) : (_Float16)0.0f;
        }
        CK(hipMemcpy(A, h.data(), (size_t)M * K * 2, hipMemcpyHostToDevice));
        CK(hipMemcpy(B, h.data(), (size_t)N * K * 2, hipMemcpyHostToDevice));
        for (int i = 0; i < 5; ++i) hipLaunchKernelGGL(probe, dim3(grid), dim3(TZ_THREADS), 0, 0, A, B, C, M, N, K);
        const int reps = 50;
        CK(hipEventRecord(e0));
        for (int i = 0; i < reps; ++i) hipLaunchKernelGGL(probe, dim3(grid), dim3(TZ_THREADS), 0, 0, A, B, C, M, N, K);
        CK(hipEventRecord(e1));
        CK(hipEventSynchronize(e1));
        float ms;
        CK(hipEventElapsedTime(&ms, e0, e1));
        const double us = ms * 1e3 / reps;
        printf("%dx%dx%d %-22s %8.2f us  %7.1f TFLOP/s  %.3f of 2500\n", M, N, K,
               random ? "operands U[-1,1):" : "operands all zero:", us, 2.0 * M * N * K / us / 1e6,
               2.0 * M * N * K / us / 1e6 / 2500.0);
    }
    return 0;
}
