// Creator.h -- name -> kernel object factories (src/Creator.h of the reference).
#pragma once
#include <string>

#include "GPTBKernel.h"
#include "MixKernel.h"
#include "ori_kernel/cp_kernel.h"
#include "ori_kernel/lbm_kernel.h"
#include "ori_kernel/mriq_kernel.h"
#include "ori_kernel/mrif_kernel.h"
#include "ori_kernel/cutcp_kernel.h"
#include "ori_kernel/fft_kernel.h"
#include "ori_kernel/hot3d_kernel.h"
#include "ori_kernel/lava_kernel.h"
#include "ori_kernel/nn_kernel.h"
#include "ori_kernel/path_kernel.h"
#include "ori_kernel/sgemm_kernel.h"
#include "ori_kernel/stencil_kernel.h"
#include "tzgemm_kernel.h"

// Memoised GPTB form of a best-effort kernel ("cp", "cutcp", "fft", "hot3d", "lava", "lbm", "mrif", "mriq", "nn", "path", "sgemm", "stencil") or
// of the GEMM ("tzgemm"); an unknown name is logger.ERROR -> exit(1).
GPTBKernel *createKernel(const std::string &name);

// Memoised fused pair of two best-effort kernels ("<a>_<b>", a < b alphabetically).
MixKernel *createMixKernel(const std::string &name);

// One fused launch object: GEMM (M,N,K already rounded) + a slice of a
// best-effort kernel, built the way TaskManager builds it for every mixed launch.
// variant "" = the kinfo default of "tzgemm_<be>".
MixKernel *createTzgemmMix(GPTBKernel *be, GPTBKernel *tz, int be_start, int be_end, int tile_start,
                           int tile_end, const std::string &variant, int launch_grid, int launch_block);

// Fused launch of two best-effort kernels (first < second alphabetically), kinfo key
// "<first>_<second>[@variant]".
MixKernel *createBePairMix(GPTBKernel *first, GPTBKernel *second, int start1, int end1, int start2, int end2,
                           const std::string &variant, int launch_grid);

// compute units of the current device (cached tkGetCuCount)
int cuCount();
