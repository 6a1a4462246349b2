// Single device translation unit of libtacker_amd.so: the natural-grid ("ori")
// kernels, their persistent-workgroup GPTB forms, the generated fused kernels,
// the small data-movement kernels of the conv->GEMM path, and the registry that
// hands all of them to the host by name.
//
// Names follow the reference: ori_<k> (src/ori_kernel/*.cu), gptb keys of
// src/main.cu:108-125 (general_ptb_* / g_general_ptb_*), <be>_tzgemm_mix
// (src/mix_kernel/tzgemm_*.cu).  Parameter lists are the reference's, so the
// host marshals arguments exactly as GPTBKernel / MixKernel do.
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>

#include "../../../include/tacker_amd.h"
#include "cp_role.h"
#include "cutcp_role.h"
#include "dnn_kernels.h"
#include "fft_role.h"
#include "hot3d_role.h"
#include "lava_role.h"
#include "lbm_role.h"
#include "mriq_role.h"
#include "nn_role.h"
#include "path_role.h"
#include "mrif_role.h"
#include "sgemm_role.h"
#include "stencil_role.h"
#include "tzgemm_role.h"
#include "tzgemm_large.h"   // the large-tile GEMM role of the 512-thread fused kernels

#define GPTB_TRAILER                                                                            \
    int grid_dimension_x, int grid_dimension_y, int grid_dimension_z, int block_dimension_x,    \
        int block_dimension_y, int block_dimension_z, int ptb_start_block_pos,                  \
        int ptb_iter_block_step, int ptb_end_block_pos, int thread_base

// ------------------------------------------------------------------ ori kernels

// grid (ceil(nx/64), ceil(ny/4)), block (32,4): wave w of the 2 takes rows 2w, 2w+1.
extern "C" __global__ __launch_bounds__(128) void ori_stencil(float c0, float c1, float *A0,
                                                              float *Anext, int nx, int ny, int nz)
{
    const int tid = threadIdx.x + threadIdx.y * blockDim.x;
    const int wave = tid >> 6;
    for (int k_first = 1; k_first <= nz - 2; k_first += STENCIL_Z_RUN)
        tk::stencil_wave_run<2, STENCIL_Z_RUN>(c0, c1, A0, Anext, nx, ny, k_first,
                                               min(STENCIL_Z_RUN, nz - 1 - k_first),
                                               blockIdx.x * 2 * STENCIL_TILE_X,
                                               blockIdx.y * STENCIL_TILE_Y + 2 * wave, tid & 63);
}

// grid (sy, sz), block sx
extern "C" __global__ void ori_lbm(float *srcGrid, float *dstGrid)
{
    const int sx = blockDim.x, sy = gridDim.x, sz = gridDim.y;
    const int c = threadIdx.x + blockIdx.x * sx + blockIdx.y * sx * sy;
    tk::lbm_cell(srcGrid, dstGrid, sx * sy * sz, c, sx, sx * sy);
}

extern "C" __global__ void ori_ComputePhiMag(float *phiR, float *phiI, float *phiMag, int numK)
{
    const int indexK = blockIdx.x * blockDim.x + threadIdx.x;
    if (indexK < numK) {
        const float real = phiR[indexK];
        const float imag = phiI[indexK];
        phiMag[indexK] = real * real + imag * imag;
    }
}

// grid numX/256, block 256
extern "C" __global__ __launch_bounds__(256) void ori_mriq(int numK, int kGlobalIndex, float *x,
                                                           float *y, float *z, float *Qr, float *Qi)
{
    (void)kGlobalIndex;
    tk::mriq_voxel(numK, x, y, z, Qr, Qi, blockIdx.x * KERNEL_Q_THREADS_PER_BLOCK + threadIdx.x);
}

extern "C" __global__ void ComputeRhoPhiGPU(int numK, float *phiR, float *phiI, float *dR, float *dI,
                                            float *realRhoPhi, float *imagRhoPhi)
{
    const int indexK = blockIdx.x * KERNEL_RHO_PHI_THREADS_PER_BLOCK + threadIdx.x;
    if (indexK < numK) {
        const float rPhiR = phiR[indexK];
        const float rPhiI = phiI[indexK];
        const float rDR = dR[indexK];
        const float rDI = dI[indexK];
        // the product on the left folded into the sum / difference, as nvcc contracts the source
        realRhoPhi[indexK] = __builtin_fmaf(rPhiR, rDR, rPhiI * rDI);
        imagRhoPhi[indexK] = __builtin_fmaf(rPhiR, rDI, -(rPhiI * rDR));
    }
}

// grid numX/256, block 256
extern "C" __global__ __launch_bounds__(256) void ori_mrif(int numK, int kGlobalIndex, float *x,
                                                           float *y, float *z, float *outR, float *outI)
{
    (void)kGlobalIndex;
    tk::mrif_voxel(numK, x, y, z, outR, outI, blockIdx.x * KERNEL_FH_THREADS_PER_BLOCK + threadIdx.x);
}

// grid (M/128, N/16), block (16,4): one wavefront where the reference has 128 threads, a lane owning the
// rows of the reference's threads l and l + 64 (src/ori_kernel/sgemm_kernel.cu:9-44)
extern "C" __global__ __launch_bounds__(64) void ori_sgemm(float *A, float *B, float *C, int NORMAL_M, int NORMAL_N,
                                                           int NORMAL_K)
{
    const int mid = threadIdx.y * blockDim.x + threadIdx.x;
    __shared__ __align__(16) float stage[64];
    tk::sgemm_thread(A, B, C, nullptr, NORMAL_M, NORMAL_N, NORMAL_K, blockIdx.x * SGEMM_TILE_M + mid,
                     blockIdx.y * SGEMM_TILE_N, 0, NORMAL_K, (tk::sgemm_lds_float *)&stage[0]);
}

// grid (regions along x, y, z), block (8,2,8): a wavefront per half region
// (src/ori_kernel/cutcp_kernel.cu:19-158; zRegionIndex_t is not read there either)
extern "C" __global__ __launch_bounds__(CUTCP_BLOCK_THREADS) void ori_cutcp(int binDim_x, int binDim_y, float *binZeroAddr,
                                                                            float h, float cutoff2, float inv_cutoff2,
                                                                            float *regionZeroAddr, int zRegionIndex_t)
{
    (void)zRegionIndex_t;
    const int tid = (threadIdx.z * blockDim.y + threadIdx.y) * blockDim.x + threadIdx.x;
    // the neighbour list in the order of the GPTB form's parts: entries p, p + parts, ... for p = 0, 1, ...
    const int len = NbrListLen;
    const int parts = max(1, (len + CUTCP_NBR_CHUNK - 1) / CUTCP_NBR_CHUNK);
    tk::cutcp_half_region<false>(binDim_x, binDim_y, binZeroAddr, h, cutoff2, inv_cutoff2, regionZeroAddr, (int)gridDim.x,
                          (int)gridDim.y, (int)blockIdx.x, (int)blockIdx.y, (int)blockIdx.z,
                          __builtin_amdgcn_readfirstlane(tid >> 6),
                          (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)), 0, parts, parts, len);
}

// grid (transforms), block 64: a wavefront per transform where the reference has a block of 128 threads
// (src/ori_kernel/fft_kernel.cu:48-61)
extern "C" __global__ __launch_bounds__(FFT_WAVE) void ori_fft(float *data)
{
    tk::fft_role<1>(data, (int)gridDim.x, (int)blockIdx.x, (int)gridDim.x, 0, (int)gridDim.x, (int)threadIdx.x, FFT_WAVE);
}

// grid (blocks of 256 records, 1), block 256 (src/ori_kernel/nn_kernel.cu:9-17)
extern "C" __global__ __launch_bounds__(NN_THREADS_PER_BLOCK) void ori_nn(LatLong *d_locations, float *d_distances,
                                                                          int numRecords, float lat, float lng)
{
    const int blocks = (int)(gridDim.x * gridDim.y);
    tk::nn_role(d_locations, d_distances, numRecords, lat, lng, (int)gridDim.x, (int)gridDim.y, (int)blockDim.x,
                (int)(gridDim.x * blockIdx.y + blockIdx.x), blocks, 0, blocks, (int)threadIdx.x, (int)blockDim.x);
}

// grid (nx/64, ny/4), block (64,4) (src/ori_kernel/hot3d_kernel.cu:9-60)
extern "C" __global__ __launch_bounds__(HOT3D_TILE_X *HOT3D_TILE_Y) void ori_hot3d(float *p, float *tIn, float *tOut,
                                                                                  float sdc, int nx, int ny, int nz,
                                                                                  float ce, float cw, float cn,
                                                                                  float cs, float ct, float cb,
                                                                                  float cc)
{
    const int blocks = (int)(gridDim.x * gridDim.y);
    tk::hot3d_role(p, tIn, tOut, sdc, nx, ny, nz, ce, cw, cn, cs, ct, cb, cc, (int)gridDim.x, (int)gridDim.y,
                   (int)blockDim.x, (int)blockDim.y, (int)(gridDim.x * blockIdx.y + blockIdx.x), blocks, 0, blocks,
                   (int)(threadIdx.y * blockDim.x + threadIdx.x), (int)(blockDim.x * blockDim.y));
}

// grid (block positions), block 64: a wavefront per position where the reference means a block of
// 256 threads (src/ori_kernel/path_kernel.cu:9-86)
extern "C" __global__ __launch_bounds__(TK_WAVE_SIZE) void ori_path(int iteration, int *gpuWall, int *gpuSrc,
                                                                    int *gpuResults, int cols, int rows, int startStep,
                                                                    int border)
{
    (void)rows;
    tk::path_role(iteration, gpuWall, gpuSrc, gpuResults, cols, startStep, border, (int)blockIdx.x, (int)gridDim.x, 0,
                  (int)gridDim.x, (int)threadIdx.x, TK_WAVE_SIZE);
}

// grid (boxes), block 64: a wavefront per home box, all 27 parts of its work, where the reference
// launches 128 threads (src/ori_kernel/lava_kernel.cu:9-141)
extern "C" __global__ __launch_bounds__(TK_WAVE_SIZE) void ori_lava(par_str d_par_gpu, dim_str d_dim_gpu,
                                                                    box_str *d_box_gpu, FOUR_VECTOR *d_rv_gpu,
                                                                    float *d_qv_gpu, FOUR_VECTOR *d_fv_gpu)
{
    tk::lava_role(d_par_gpu, d_dim_gpu, d_box_gpu, d_rv_gpu, d_qv_gpu, d_fv_gpu, (int)gridDim.x, (int)blockIdx.x,
                  (int)gridDim.x, 0, (int)gridDim.x * LAVA_PARTS, (int)threadIdx.x, TK_WAVE_SIZE);
}

// Values that depend on (index, seed) only, for the default instances of the large kernels.
__device__ __forceinline__ unsigned tk_fill_hash(unsigned long long i, unsigned seed)
{
    unsigned x = (unsigned)i ^ ((unsigned)(i >> 32) * 0x9E3779B9u) ^ seed;
    x ^= x >> 16;
    x *= 0x7feb352du;
    x ^= x >> 15;
    x *= 0x846ca68bu;
    x ^= x >> 16;
    return x;
}
extern "C" __global__ __launch_bounds__(256) void tk_fill_uniform(float *dst, unsigned long long n, unsigned seed,
                                                                  float lo, float hi)
{
    const unsigned long long stride = (unsigned long long)gridDim.x * blockDim.x;
    for (unsigned long long i = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        dst[i] = lo + (hi - lo) * ((float)(tk_fill_hash(i, seed) >> 8) * (1.0f / 16777216.0f));
}
extern "C" __global__ __launch_bounds__(256) void tk_fill_int_mod(int *dst, unsigned long long n, unsigned seed,
                                                                  int mod)
{
    const unsigned long long stride = (unsigned long long)gridDim.x * blockDim.x;
    for (unsigned long long i = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride)
        dst[i] = (int)(tk_fill_hash(i, seed) % (unsigned)mod);
}

// grid (volx/128, voly/8), block (16,8)
extern "C" __global__ __launch_bounds__(128) void ori_cp(int numatoms, float gridspacing,
                                                         float *energygrid)
{
    tk::cp_block(numatoms, gridspacing, energygrid, blockIdx.x, blockIdx.y, gridDim.x, threadIdx.x,
                 threadIdx.y);
}

// ------------------------------------------------------------------ GPTB kernels

// general_ptb_<kernel> (g_general_ptb_ for mriq and cp): written by fusion/code/gen_run.py from the
// same role descriptions as the fused kernels
#include "../gptb_kernel/gptb_kernels.inc"

// ---- tzgemm for callers that cannot allocate device memory --------------------------------
// The same role with its workspace handed in as an argument, and the workspace itself: a
// file-scope array every GPU the library runs on holds until the process ends.  TZ_SCRATCH_BYTES
// covers the largest workspace any shape needs (512 partial tiles of 16 KiB + the counters).
// `scratch` is a host-side stand-in in host code, never a device address: host code uses the
// address hipGetSymbolAddress gave for the current device (tk_scratch_setup / tk_tzgemm_scratch).
static __device__ __align__(256) unsigned char scratch[TZ_SCRATCH_BYTES];

extern "C" __global__ __launch_bounds__(TZ_THREADS) __attribute__((amdgpu_waves_per_eu(1, 1))) void general_ptb_tzgemm_scratch(
    _Float16 *A, _Float16 *B, float *C, int M_GLOBAL, int N_GLOBAL, int K_GLOBAL, unsigned *workspace, GPTB_TRAILER)
{
    __shared__ __align__(16) char tz_lds[TZ_LDS_BYTES];
    tk::WorkgroupSync sync;
    tk::tzgemm_role<TZ_STAGES>(A, B, C, M_GLOBAL, N_GLOBAL, K_GLOBAL, workspace, (int)blockIdx.x, ptb_iter_block_step,
                    ptb_start_block_pos, ptb_end_block_pos, (int)threadIdx.x - thread_base, tz_lds,
                    sync);
}

// zeroes n 32-bit words (the arrival counters at the head of the workspace); a kernel rather
// than a memset so that the call can be recorded into a HIP graph
extern "C" __global__ void tz_clear_words(unsigned *words, int n)
{
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) words[i] = 0u;
}

namespace {
constexpr int kMaxDevices = 64;
void *g_scratch_address[kMaxDevices];   // address of `scratch` on each device that was set up
}

// Once per device, with that device current (tkInit calls it): the device address of the array.
extern "C" int tk_scratch_setup(int device)
{
    if (device < 0 || device >= kMaxDevices) return TK_ERROR_INVALID_VALUE;
    if (g_scratch_address[device]) return TK_SUCCESS;
    void *ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || !ptr) {
        (void)hipGetLastError();
        return TK_ERROR_DEVICE;
    }
    g_scratch_address[device] = ptr;
    return TK_SUCCESS;
}

// The current device's copy of the array and its size; fails if the device was never set up.
extern "C" int tk_tzgemm_scratch(void **ptr, size_t *bytes)
{
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices || !g_scratch_address[device])
        return TK_ERROR_INVALID_VALUE;
    *ptr = g_scratch_address[device];
    *bytes = sizeof(scratch);
    return TK_SUCCESS;
}

// Counts the floats with bit patterns in [lo_bits, hi_bits) for which the short form of
// 1 / sqrt (tk::cp_inv_sqrt_short) differs from 1.0f / sqrtf(x) in any bit.
extern "C" __global__ void cp_inv_sqrt_selftest(unsigned lo_bits, unsigned hi_bits,
                                                unsigned long long *mismatches)
{
    unsigned long long bad = 0;
    for (unsigned long long b = (unsigned long long)lo_bits + blockIdx.x * (unsigned long long)blockDim.x + threadIdx.x;
         b < hi_bits; b += (unsigned long long)gridDim.x * blockDim.x) {
        const float x = __uint_as_float((unsigned)b);
        bad += __float_as_uint(tk::cp_inv_sqrt_short(x)) != __float_as_uint(1.0f / sqrtf(x));
    }
    if (bad) atomicAdd(mismatches, bad);
}

// ------------------------------------------------------------------ conv -> GEMM helpers

// Caffe im2col, NCHW (src/TaskManager.cu:48-82): grid-stride over
// channels*height_col*width_col work items.
extern "C" __global__ void im2col_gpu_kernel_(int n, float *data_im, int height, int width,
                                              int kernel_h, int kernel_w, int pad_h, int pad_w,
                                              int stride_h, int stride_w, int dilation_h,
                                              int dilation_w, int height_col, int width_col,
                                              float *data_col, int data_im_size, int data_col_size)
{
    (void)data_im_size;
    (void)data_col_size;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += blockDim.x * gridDim.x) {
        const int h_index = i / width_col;
        const int h_col = h_index % height_col;
        const int w_col = i % width_col;
        const int c_im = h_index / height_col;
        const int c_col = c_im * kernel_h * kernel_w;
        const int h_offset = h_col * stride_h - pad_h;
        const int w_offset = w_col * stride_w - pad_w;
        float *data_col_ptr = data_col + ((size_t)c_col * height_col + h_col) * width_col + w_col;
        const float *data_im_ptr = data_im + ((long)c_im * height + h_offset) * width + w_offset;
        for (int ki = 0; ki < kernel_h; ++ki) {
            for (int kj = 0; kj < kernel_w; ++kj) {
                const int h_im = h_offset + ki * dilation_h;
                const int w_im = w_offset + kj * dilation_w;
                *data_col_ptr = (h_im >= 0 && w_im >= 0 && h_im < height && w_im < width)
                                    ? data_im_ptr[ki * dilation_h * width + kj * dilation_w]
                                    : 0.0f;
                data_col_ptr += (size_t)height_col * width_col;
            }
        }
    }
}

// src/TaskManager.cu:85-90
extern "C" __global__ void convertFp32ToFp16_(_Float16 *out, float *in, int n)
{
    const int idx = blockDim.x * blockIdx.x + threadIdx.x;
    if (idx < n) out[idx] = (_Float16)in[idx];
}

// ------------------------------------------------------------------ fused kernels (generated)
#include "../mix_kernel/mix_kernels.inc"

// ------------------------------------------------------------------ registry
extern "C" void tk_register_large_kernels(tk_kernel_insert_fn insert, void *ctx);   // tzgemm_large.hip

extern "C" TK_API int tk_register_kernels(tk_kernel_insert_fn insert, void *ctx)
{
    if (!insert) return TK_ERROR_INVALID_VALUE;
    insert("ori_stencil", (const void *)ori_stencil, ctx);
    insert("ori_lbm", (const void *)ori_lbm, ctx);
    insert("ori_ComputePhiMag", (const void *)ori_ComputePhiMag, ctx);
    insert("ori_mriq", (const void *)ori_mriq, ctx);
    insert("ori_cp", (const void *)ori_cp, ctx);
    insert("ComputeRhoPhiGPU", (const void *)ComputeRhoPhiGPU, ctx);
    insert("ori_mrif", (const void *)ori_mrif, ctx);
    insert("ori_sgemm", (const void *)ori_sgemm, ctx);
    insert("ori_fft", (const void *)ori_fft, ctx);
    insert("ori_cutcp", (const void *)ori_cutcp, ctx);
    insert("ori_nn", (const void *)ori_nn, ctx);
    insert("ori_hot3d", (const void *)ori_hot3d, ctx);
    insert("ori_path", (const void *)ori_path, ctx);
    insert("ori_lava", (const void *)ori_lava, ctx);
    insert("fill_uniform", (const void *)tk_fill_uniform, ctx);
    insert("fill_int_mod", (const void *)tk_fill_int_mod, ctx);
    insert("gptb_tzgemm_scratch", (const void *)general_ptb_tzgemm_scratch, ctx);
    insert("tz_clear_words", (const void *)tz_clear_words, ctx);
    insert("cp_inv_sqrt_selftest", (const void *)cp_inv_sqrt_selftest, ctx);
    insert("im2col", (const void *)im2col_gpu_kernel_, ctx);
    insert("convert_fp32_to_fp16", (const void *)convertFp32ToFp16_, ctx);
    insert("im2col_nhwc_f16", (const void *)im2col_nhwc_f16, ctx);
    insert("im2col3x3_scatter_nhwc_f16", (const void *)im2col3x3_scatter_nhwc_f16, ctx);
    insert("maxpool2x2_nhwc", (const void *)maxpool2x2_nhwc, ctx);
    insert("pack_fc_input", (const void *)pack_fc_input, ctx);
    insert("pack_fc_input_pooled", (const void *)pack_fc_input_pooled, ctx);
    tk_register_gptb_kernels(insert, ctx);
    tk_register_mix_kernels(insert, ctx);
    tk_register_large_kernels(insert, ctx);
    return TK_SUCCESS;
}

// Device symbols the host fills by name (cudaMemcpyToSymbol in the reference).
extern "C" int tk_device_symbol(const char *name, const void **symbol, size_t *bytes)
{
    if (!name) return TK_ERROR_INVALID_VALUE;
    if (__builtin_strcmp(name, "ck") == 0) {
        *symbol = (const void *)&ck;
        *bytes = sizeof(ck);
        return TK_SUCCESS;
    }
    if (__builtin_strcmp(name, "c_mrif") == 0) {
        *symbol = (const void *)&c_mrif;
        *bytes = sizeof(c_mrif);
        return TK_SUCCESS;
    }
    if (__builtin_strcmp(name, "atominfo") == 0) {
        *symbol = (const void *)&atominfo;
        *bytes = sizeof(atominfo);
        return TK_SUCCESS;
    }
    if (__builtin_strcmp(name, "NbrListLen") == 0) {
        *symbol = (const void *)&NbrListLen;
        *bytes = sizeof(NbrListLen);
        return TK_SUCCESS;
    }
    if (__builtin_strcmp(name, "NbrList") == 0) {
        *symbol = (const void *)&NbrList;
        *bytes = sizeof(NbrList);
        return TK_SUCCESS;
    }
    if (__builtin_strcmp(name, "tz_ws_table") == 0) {
        *symbol = (const void *)&tz_ws_table;
        *bytes = sizeof(tz_ws_table);
        return TK_SUCCESS;
    }
    if (__builtin_strcmp(name, "tk_spin_fail") == 0) {
        *symbol = (const void *)&tk_spin_fail;
        *bytes = sizeof(tk_spin_fail);
        return TK_SUCCESS;
    }
    return TK_ERROR_NOT_FOUND;
}
