// fused_probe.hip -- the wave-split fused kernel of tzgemm 2048^3 + stencil 512x512x64 (the body
// the generator emits as stencil_tzgemm_mix_wave_512) in a plain HIP program, with two additions:
// each role's first wave of every workgroup writes the wall clock when the role starts and when
// it ends, and the GEMM role can be built without the loads (TZ_KNOCK_OUT_LOADS) or without the
// MFMAs (TZ_KNOCK_OUT_MFMA) of its steady K loop (results wrong on purpose).  It prints the time
// of the fused launch, of each role alone in the same kernel (the other role's range empty), and
// when the roles of the fused launch finish.
//
//   build: hipcc --offload-arch=gfx950 -O3 -std=c++17 -ffp-contract=off -Xclang -target-feature
//          -Xclang -packed-fp32-ops -mllvm -amdgpu-mfma-vgpr-form [-DTZ_KNOCK_OUT_...] -o fused_probe fused_probe.hip
//   run:   ./fused_probe
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <vector>

#include "../kernels/stencil_role.h"
#include "../kernels/tzgemm_role.h"

#define CK(x)                                                                          \
    do {                                                                               \
        hipError_t e_ = (x);                                                           \
        if (e_ != hipSuccess) {                                                        \
            printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);      \
            exit(1);                                                                   \
        }                                                                              \
    } while (0)

// stamps[4 * workgroup + {0,1,2,3}] = GEMM role start, end, stencil role start, end (100 MHz ticks)
__global__ __launch_bounds__(768) void fused(float c0, float c1, float *A0, float *Anext, int nx, int ny, int nz, int gx, int gy,
                                            int gz, int be_start, int be_end, _Float16 *A, _Float16 *B, float *C, int M,
                                            int N, int K, int tile_start, int tile_end, unsigned long long *stamps)
{
    __shared__ __align__(16) char tz_lds[TZ_LDS_BYTES + 16];
    unsigned *tz_arrivals = reinterpret_cast<unsigned *>(tz_lds + TZ_LDS_BYTES);
    if (threadIdx.x == 0) *tz_arrivals = 0u;
    __syncthreads();
    const bool stamper = (threadIdx.x & 255) == 0 && threadIdx.x < 512;   // thread 0 (GEMM), 256 (stencil)
    unsigned long long *mine = stamps + 4 * blockIdx.x + (threadIdx.x < 256 ? 0 : 2);
    if (stamper) mine[0] = wall_clock64();
    if (threadIdx.x < 256) {
        __builtin_amdgcn_s_setprio(TK_GEMM_WAVE_PRIORITY);
        tk::RoleSpinSync sync(tz_arrivals, 4, &tk_spin_fail);
        tk::tzgemm_role<TZ_STAGES, false>(A, B, C, M, N, K, nullptr, (int)blockIdx.x, (int)gridDim.x, tile_start, tile_end,
                                          (int)threadIdx.x, tz_lds, sync);
    } else {
        tk::stencil_role(c0, c1, A0, Anext, nx, ny, nz, gx, gy, gz, (int)blockIdx.x, (int)gridDim.x, be_start, be_end,
                         (int)threadIdx.x - 256, 512);
    }
    if (stamper) mine[1] = wall_clock64();
}

int main()
{
    const int M = 2048, N = 2048, K = 2048, nx = 512, ny = 512, nz = 64;
    const int gx = (nx + 2 * STENCIL_TILE_X - 1) / (2 * STENCIL_TILE_X), gy = (ny + STENCIL_TILE_Y - 1) / STENCIL_TILE_Y, gz = (nz - 2 + STENCIL_Z_RUN - 1) / STENCIL_Z_RUN;
    const int positions = gx * gy * gz, tiles = (M / 64) * (N / 64), grid = 256;
    _Float16 *A, *B;
    float *C, *g0, *g1;
    unsigned long long *stamps;
    CK(hipMalloc(&A, (size_t)M * K * 2));
    CK(hipMalloc(&B, (size_t)N * K * 2));
    CK(hipMalloc(&C, (size_t)M * N * 4));
    CK(hipMalloc(&g0, (size_t)nx * ny * nz * 4));
    CK(hipMalloc(&g1, (size_t)nx * ny * nz * 4));
    CK(hipMalloc(&stamps, grid * 4 * sizeof(unsigned long long)));
    {
        std::vector<_Float16> h((size_t)M * K);
        unsigned s = 12345u;
        for (auto &v : h) {
            s = s * 1664525u + 1013904223u;
            v = (_Float16)(((s >> 8) & 0xFFFF) / 32768.0f - 1.0f);
        }
        CK(hipMemcpy(A, h.data(), h.size() * 2, hipMemcpyHostToDevice));
        CK(hipMemcpy(B, h.data(), h.size() * 2, hipMemcpyHostToDevice));
        std::vector<float> g((size_t)nx * ny * nz);
        for (auto &v : g) {
            s = s * 1664525u + 1013904223u;
            v = (s >> 8) / 16777216.0f;
        }
        CK(hipMemcpy(g0, g.data(), g.size() * 4, hipMemcpyHostToDevice));
        CK(hipMemcpy(g1, g.data(), g.size() * 4, hipMemcpyHostToDevice));
    }
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    const float c0 = 1.0f / 6.0f, c1 = 1.0f / 36.0f;
    struct Case { const char *name; int be_end, tile_end; } cases[3] = {
        {"both roles", positions, tiles}, {"GEMM role alone", 0, tiles}, {"stencil role alone", positions, 0}};
    for (const Case &cs : cases) {
        const int reps = 100;
        for (int i = 0; i < 5; ++i)
            hipLaunchKernelGGL(fused, dim3(grid), dim3(768), 0, 0, c0, c1, g0, g1, nx, ny, nz, gx, gy, gz, 0, cs.be_end, A, B, C,
                               M, N, K, 0, cs.tile_end, stamps);
        CK(hipEventRecord(e0));
        for (int i = 0; i < reps; ++i)
            hipLaunchKernelGGL(fused, dim3(grid), dim3(768), 0, 0, c0, c1, g0, g1, nx, ny, nz, gx, gy, gz, 0, cs.be_end, A, B, C,
                               M, N, K, 0, cs.tile_end, stamps);
        CK(hipEventRecord(e1));
        CK(hipEventSynchronize(e1));
        float ms;
        CK(hipEventElapsedTime(&ms, e0, e1));
        std::vector<unsigned long long> h(grid * 4);
        CK(hipMemcpy(h.data(), stamps, h.size() * sizeof(unsigned long long), hipMemcpyDeviceToHost));
        unsigned long long first = ~0ull;
        for (int w = 0; w < grid; ++w) first = std::min(first, std::min(h[4 * w], h[4 * w + 2]));
        std::vector<double> gemm_end, st_end;
        for (int w = 0; w < grid; ++w) {
            gemm_end.push_back((h[4 * w + 1] - first) * 0.01);   // 100 MHz ticks -> us
            st_end.push_back((h[4 * w + 3] - first) * 0.01);
        }
        std::sort(gemm_end.begin(), gemm_end.end());
        std::sort(st_end.begin(), st_end.end());
        printf("%-20s %7.2f us per launch; last launch: GEMM role ends at %5.1f / %5.1f / %5.1f us (first, median, last "
               "workgroup), stencil role at %5.1f / %5.1f / %5.1f us\n",
               cs.name, ms * 1e3 / reps, gemm_end.front(), gemm_end[grid / 2], gemm_end.back(), st_end.front(),
               st_end[grid / 2], st_end.back());
    }
    return 0;
}
