// feed_rate.hip -- how fast a CU can pull GEMM operand panels from L2 / HBM into LDS with
// LDS-direct loads (global_load_lds_dwordx4), by the number of contiguous bytes a load takes
// from each matrix row.  Every workgroup (one per CU, 4 waves) plays one 256 x 256 tile of a
// 4096 x 4096 x 4096 fp16 GEMM: it walks k through the 256 rows of its A panel and the 256 rows
// of its B panel (row pitch 8192 bytes) and moves SEG bytes of every row per step, the way the
// K loop of a tile does, with no arithmetic.  16 workgroups share each panel, as the tiles of a
// GEMM do.
//
//   build: hipcc --offload-arch=gfx950 -O3 -o feed_rate feed_rate.hip
//   run:   ./feed_rate
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

#define CK(x)                                                                          \
    do {                                                                               \
        hipError_t e_ = (x);                                                           \
        if (e_ != hipSuccess) {                                                        \
            printf("HIP error %s at line %d\n", hipGetErrorString(e_), __LINE__);      \
            exit(1);                                                                   \
        }                                                                              \
    } while (0)

typedef __attribute__((address_space(1))) const void *gptr_t;
typedef __attribute__((address_space(3))) void *lptr_t;

constexpr int DIM = 4096;          // M = N = K
constexpr int PITCH = DIM * 2;     // bytes per matrix row
constexpr int ROWS = 512;          // rows a tile pulls per step: 256 of A, 256 of B

// SEG bytes per row and step; one load instruction covers 1024 / SEG rows
template <int SEG>
__global__ __launch_bounds__(256) void feed(const char *A, const char *B, float *sink, int in_flight)
{
    __shared__ __attribute__((aligned(16))) char lds[4 * 32768];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    constexpr int LANES_PER_ROW = SEG / 16;
    constexpr int ROWS_PER_LOAD = 64 / LANES_PER_ROW;
    constexpr int LOADS = ROWS / ROWS_PER_LOAD / 4;           // per wave and step
    constexpr int STEPS = PITCH / SEG;
    const char *a_panel = A + (size_t)(blockIdx.x / 16) * 256 * PITCH;
    const char *b_panel = B + (size_t)(blockIdx.x % 16) * 256 * PITCH;
    const unsigned lane_off = (unsigned)((lane / LANES_PER_ROW) * PITCH + (lane % LANES_PER_ROW) * 16);
    int group = 0;                                            // groups of 8 loads = 32 KiB per workgroup
    for (int s = 0; s < STEPS; ++s) {
#pragma unroll
        for (int j = 0; j < LOADS; ++j) {
            const int row = (j * 4 + wave) * ROWS_PER_LOAD;    // of the 512
            const char *src = (row < 256 ? a_panel + (size_t)row * PITCH : b_panel + (size_t)(row - 256) * PITCH) +
                              (size_t)s * SEG + lane_off;
            __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(lds + (group & 3) * 32768 + ((j & 7) * 4 + wave) * 1024),
                                             16, 0, 0);
            if ((j & 7) == 7) {
                // keep in_flight groups of loads outstanding, as a ring of stages does
                if (in_flight == 1) __builtin_amdgcn_s_waitcnt(0x0F70 | 8);
                else if (in_flight == 2) __builtin_amdgcn_s_waitcnt(0x4F70 | 0);   // vmcnt(16)
                else __builtin_amdgcn_s_waitcnt(0x4F70 | 8);                       // vmcnt(24)
                ++group;
            }
        }
    }
    __builtin_amdgcn_s_waitcnt(0x0F70);
    __syncthreads();
    if (*reinterpret_cast<float *>(lds + threadIdx.x * 4) == 12345.f) sink[0] = 1.f;
}

template <int SEG>
void run(const char *A, const char *B, float *sink, int in_flight)
{
    hipEvent_t e0, e1;
    CK(hipEventCreate(&e0));
    CK(hipEventCreate(&e1));
    float best = 1e9f;
    for (int rep = 0; rep < 5; ++rep) {
        CK(hipEventRecord(e0));
        hipLaunchKernelGGL(feed<SEG>, dim3(256), dim3(256), 0, 0, A, B, sink, in_flight);
        CK(hipEventRecord(e1));
        CK(hipEventSynchronize(e1));
        float ms;
        CK(hipEventElapsedTime(&ms, e0, e1));
        if (rep > 0 && ms < best) best = ms;
    }
    const double bytes_per_cu = (double)ROWS * PITCH;
    printf("%4d bytes per row and load, %d x 32 KiB in flight per CU: %8.1f us  %6.1f GB/s per CU  %6.2f TB/s all CUs\n", SEG,
           in_flight, best * 1e3, bytes_per_cu / (best * 1e-3) / 1e9, 256 * bytes_per_cu / (best * 1e-3) / 1e12);
}

int main()
{
    char *A, *B;
    float *sink;
    CK(hipMalloc(&A, (size_t)DIM * PITCH));
    CK(hipMalloc(&B, (size_t)DIM * PITCH));
    CK(hipMalloc(&sink, 64));
    CK(hipMemset(A, 1, (size_t)DIM * PITCH));
    CK(hipMemset(B, 2, (size_t)DIM * PITCH));
    for (int in_flight = 1; in_flight <= 3; ++in_flight) {
        run<64>(A, B, sink, in_flight);
        run<128>(A, B, sink, in_flight);
        run<256>(A, B, sink, in_flight);
        run<512>(A, B, sink, in_flight);
    }
    return 0;
}
