// Second device translation unit of libtacker_amd.so: the stand-alone tzgemm kernel in its
// large-tile form (tzgemm_large.h).  It is compiled apart from kernels.hip because it needs the
// other half of the register file: its 256 accumulator registers live in AGPRs, while every
// other kernel is built with MFMA results in arch VGPRs (-amdgpu-mfma-vgpr-form).
//
// Parameter list = general_ptb_tzgemm's (src/gptb_kernel/tzgemm_kernel.cu:430-433): the host
// launches this kernel instead of general_ptb_tzgemm for the shapes tz_use_large names
// (OriTZGEMMKernel::funcVariant), with the same arguments.
#include <hip/hip_runtime.h>

#include "../../../include/tacker_amd.h"
#include "tzgemm_large.h"

extern "C" __global__ __launch_bounds__(TZ_THREADS) __attribute__((amdgpu_waves_per_eu(1, 1))) void general_ptb_tzgemm_large(
    _Float16 *A, _Float16 *B, float *C, int M_GLOBAL, int N_GLOBAL, int K_GLOBAL, int grid_dimension_x,
    int grid_dimension_y, int grid_dimension_z, int block_dimension_x, int block_dimension_y, int block_dimension_z,
    int ptb_start_block_pos, int ptb_iter_block_step, int ptb_end_block_pos, int thread_base)
{
    (void)grid_dimension_x;
    (void)grid_dimension_y;
    (void)grid_dimension_z;
    (void)block_dimension_x;
    (void)block_dimension_y;
    (void)block_dimension_z;
    __shared__ __align__(16) char tz_lds[TZ_LDS_BYTES];
    // a launch on a shape the form does not cover (the host never makes one) computes nothing
    if (M_GLOBAL % TZ_LARGE_TILE || N_GLOBAL % TZ_LARGE_TILE || K_GLOBAL % 128) return;
    tk::WorkgroupSync sync;
    tk::tzgemm_role_large<8, 8>(A, B, C, M_GLOBAL, N_GLOBAL, K_GLOBAL, (int)blockIdx.x, ptb_iter_block_step,
                                ptb_start_block_pos, ptb_end_block_pos, (int)threadIdx.x - thread_base, tz_lds,
                                (size_t)M_GLOBAL * (size_t)N_GLOBAL * sizeof(float) > TZ_LARGE_STREAM_C_BYTES, sync);
}

extern "C" void tk_register_large_kernels(tk_kernel_insert_fn insert, void *ctx)
{
    insert("gptb_tzgemm@large", (const void *)general_ptb_tzgemm_large, ctx);
}
