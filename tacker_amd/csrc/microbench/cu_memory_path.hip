// cu_memory_path.hip -- what one CU's vector-memory path moves when every CU streams from
// L2-resident data, by kind of access, and what a workgroup gets that does two kinds at once the
// way a wave-split fused kernel does (4 waves of LDS-direct loads, 8 waves of vector loads and
// stores).
//
//   build: hipcc --offload-arch=gfx950 -O3 -o cu_memory_path cu_memory_path.hip
//   run:   ./cu_memory_path
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

typedef __attribute__((address_space(1))) const void *gptr_t;
typedef __attribute__((address_space(3))) void *lptr_t;
typedef float float4_t __attribute__((ext_vector_type(4)));
#define CK(x)                                                                          \
    do {                                                                               \
        hipError_t e_ = (x);                                                           \
        if (e_ != hipSuccess) {                                                        \
            printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);      \
            exit(1);                                                                   \
        }                                                                              \
    } while (0)

// each workgroup (256 threads) streams iters x 32 KiB out of (or into) a 1 MiB window
// MODE 0 LDS-direct dwordx4 loads, 1 dwordx4 loads to registers, 2 dwordx4 stores, 3 dword loads
template <int MODE>
__global__ __launch_bounds__(256) void one_kind(char *src, float *sink, int iters)
{
    __shared__ __attribute__((aligned(16))) char lds[65536];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    char *base = src + (size_t)(blockIdx.x % 64) * (1 << 20);
    float4_t acc = {0, 0, 0, 0};
    for (int it = 0; it < iters; ++it) {
        char *p = base + (size_t)(it & 31) * 32768 + wave * 8192 + lane * 16;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            if (MODE == 0)
                __builtin_amdgcn_global_load_lds((gptr_t)(p + j * 1024),
                                                 (lptr_t)(lds + (it & 1) * 32768 + wave * 8192 + j * 1024), 16, 0, 0);
            else if (MODE == 1)
                acc += *reinterpret_cast<const float4_t *>(p + j * 1024);
            else if (MODE == 2)
                *reinterpret_cast<float4_t *>(p + j * 1024) = acc;
            else {
                const char *q = base + (size_t)(it & 31) * 32768 + wave * 8192 + j * 1024 + lane * 4;
                acc.x += *reinterpret_cast<const float *>(q);
                acc.y += *reinterpret_cast<const float *>(q + 256);
                acc.z += *reinterpret_cast<const float *>(q + 512);
                acc.w += *reinterpret_cast<const float *>(q + 768);
            }
        }
        if (MODE == 0 && (it & 3) == 3) __builtin_amdgcn_s_waitcnt(0x0F70 | 8);   // vmcnt(8)
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    if (MODE == 0) acc.x = *reinterpret_cast<float *>(lds + threadIdx.x * 4);
    if (acc.x + acc.y + acc.z + acc.w == 12345.f) sink[0] = acc.x;
}

// 12 waves per workgroup: waves 0-3 stream dma_iters x 32 KiB with LDS-direct loads, waves 4-11
// vec_iters x (64 KiB of loads + 32 KiB of stores) with float4 accesses
__global__ __launch_bounds__(768) void two_kinds(const char *src, char *dst, float *sink, int dma_iters, int vec_iters)
{
    __shared__ __attribute__((aligned(16))) char lds[65536];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const char *base = src + (size_t)(blockIdx.x % 32) * (1 << 20);
    float4_t acc = {0, 0, 0, 0};
    if (wave < 4) {
        for (int it = 0; it < dma_iters; ++it) {
            const char *p = base + (size_t)(it & 15) * 32768 + wave * 8192 + lane * 16;
#pragma unroll
            for (int j = 0; j < 8; ++j)
                __builtin_amdgcn_global_load_lds((gptr_t)(p + j * 1024),
                                                 (lptr_t)(lds + (it & 1) * 32768 + wave * 8192 + j * 1024), 16, 0, 0);
            if ((it & 3) == 3) __builtin_amdgcn_s_waitcnt(0x0F70 | 8);
        }
        __builtin_amdgcn_s_waitcnt(0x0F70);
    } else {
        const int w = wave - 4;
        char *out = dst + (size_t)(blockIdx.x % 32) * (1 << 20);
        for (int it = 0; it < vec_iters; ++it) {
            const char *p = base + (1 << 19) + (size_t)(it & 7) * 65536 + w * 8192 + lane * 16;
            float4_t s = {0, 0, 0, 0};
#pragma unroll
            for (int j = 0; j < 8; ++j) s += *reinterpret_cast<const float4_t *>(p + j * 1024);
            acc += s;
#pragma unroll
            for (int j = 0; j < 4; ++j)
                *reinterpret_cast<float4_t *>(out + (size_t)(it & 7) * 32768 + w * 4096 + j * 1024 + lane * 16) = s;
        }
    }
    if (acc.x + acc.y + acc.z + acc.w == 12345.f) sink[0] = acc.x;
}

template <int MODE>
void run_one(const char *name, char *src, float *sink)
{
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    const int iters = 2048, grid = 256;
    float best = 1e9f;
    for (int rep = 0; rep < 4; ++rep) {
        CK(hipEventRecord(e0));
        hipLaunchKernelGGL(one_kind<MODE>, dim3(grid), dim3(256), 0, 0, src, sink, iters);
        CK(hipEventRecord(e1));
        CK(hipEventSynchronize(e1));
        float ms;
        CK(hipEventElapsedTime(&ms, e0, e1));
        if (rep > 0 && ms < best) best = ms;
    }
    const double bytes = (double)grid * iters * 32768;
    printf("%-32s %7.3f ms  %5.1f TB/s all CUs, %6.1f GB/s per CU\n", name, best, bytes / best / 1e9, bytes / best / 1e6 / grid);
}

int main()
{
    char *src, *dst;
    float *sink;
    CK(hipMalloc(&src, 64 << 20));
    CK(hipMemset(src, 0, 64 << 20));
    CK(hipMalloc(&dst, 32 << 20));
    CK(hipMalloc(&sink, 64));
    run_one<0>("global_load_lds_dwordx4", src, sink);
    run_one<1>("global_load_dwordx4 -> VGPR", src, sink);
    run_one<2>("global_store_dwordx4", src, sink);
    run_one<3>("global_load_dword x 4", src, sink);
    // per CU and "tile": 1 MiB of LDS-direct loads (32 x 32 KiB, a 128x128x2048 GEMM tile) and
    // 448 KiB of loads + 224 KiB of stores (7 x (64 + 32) KiB, a stencil share), alone and together
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    const int scale = 64;
    const int cfg[3][2] = {{32 * scale, 0}, {0, 7 * scale}, {32 * scale, 7 * scale}};
    const char *what[3] = {"LDS-direct loads alone (4 waves)", "vector loads + stores alone (8 waves)", "both in one workgroup"};
    for (int c = 0; c < 3; ++c) {
        float best = 1e9f;
        for (int rep = 0; rep < 3; ++rep) {
            CK(hipEventRecord(e0));
            hipLaunchKernelGGL(two_kinds, dim3(256), dim3(768), 0, 0, src, dst, sink, cfg[c][0], cfg[c][1]);
            CK(hipEventRecord(e1));
            CK(hipEventSynchronize(e1));
            float ms;
            CK(hipEventElapsedTime(&ms, e0, e1));
            if (rep > 0 && ms < best) best = ms;
        }
        printf("%-40s %6.1f us per tile\n", what[c], best * 1e3 / scale);
    }
    return 0;
}
