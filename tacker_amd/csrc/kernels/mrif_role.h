// MRI-FHD role: FhD(x) += sum_k RhoPhi_k * exp(i 2 pi k.x), RhoPhi = conj(phi) * d.
//
// Replaces ComputeRhoPhiGPU / ori_mrif / general_ptb_mrif
// (src/ori_kernel/mrif_kernel.cu:62-152, src/gptb_kernel/mrif_kernel.cu:6-170).
// Kept: one thread per voxel, blocks of 256 voxels, read-modify-write of
// outR/outI, the k table as an array of {Kx,Ky,Kz,RhoPhiR,RhoPhiI} in constant
// memory, fp32 order
//   arg = 2pi * ((Kx*x + Ky*y) + Kz*z)
//   outR += RhoPhiR*cos(arg) - RhoPhiI*sin(arg);  outI += RhoPhiI*cos(arg) + RhoPhiR*sin(arg)
// with k ascending.  The reference's loop "for FHGrid < 1" handles only the first
// 256-sample grid of the table; here all numK samples held in the table are used.
//
// The kernel has the shape of MRI-Q (a voxel block times a run of k records) and
// shares its walk over block positions (mriq_role.h): x = blocks of 256 voxels,
// y = chunks of MRIF_K_CHUNK records, one owner thread group per voxel block.
// As there, the hardware sine and cosine take the phase in revolutions, and the
// multiply-adds are fused the way the reference's source contracts under nvcc's
// default -fmad=true: the product on the left of each sum or difference is
// folded into it, fma(RhoPhiR, cos, -(RhoPhiI*sin)) and fma(RhoPhiI, cos,
// RhoPhiR*sin), and the result is then added to the running value.
#pragma once
#include "mriq_role.h"
#include "../header/mrif_header.h"

__constant__ mrif_kValues c_mrif[MRIF_MAX_K];

namespace tk {

static_assert(MRIF_K_CHUNK == MRIQ_K_CHUNK && KERNEL_FH_THREADS_PER_BLOCK == KERNEL_Q_THREADS_PER_BLOCK,
              "MRI-FHD shares MRI-Q's position grid: same voxel block and k chunk");

template <int V>
__device__ __forceinline__ void mrif_voxels(int k_begin, int k_end, const float *__restrict__ x,
                                            const float *__restrict__ y, const float *__restrict__ z,
                                            float *__restrict__ outR, float *__restrict__ outI,
                                            const int (&xIndex)[V])
{
    float sX[V], sY[V], sZ[V], sOutR[V], sOutI[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
        const int i = xIndex[v];
        sX[v] = x[i];
        sY[v] = y[i];
        sZ[v] = z[i];
        sOutR[v] = outR[i];
        sOutI[v] = outI[i];
    }
    // U records at a time, stage by stage, as in mriq_voxels: the U * V chains are independent
    // until the accumulation, which runs in ascending k.
    constexpr int U = 4;
    int kIndex = k_begin;
    for (; kIndex + U <= k_end; kIndex += U) {
        mrif_kValues k[U];
#pragma unroll
        for (int u = 0; u < U; ++u) k[u] = c_mrif[kIndex + u];
        float c[U][V], s[U][V];
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int v = 0; v < V; ++v) {
                const float phase = __builtin_fmaf(k[u].Kz, sZ[v], __builtin_fmaf(k[u].Ky, sY[v], k[u].Kx * sX[v]));
                c[u][v] = __builtin_amdgcn_fractf(phase);   // revolutions
            }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int v = 0; v < V; ++v) {
                s[u][v] = __builtin_amdgcn_sinf(c[u][v]);
                c[u][v] = __builtin_amdgcn_cosf(c[u][v]);
            }
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int v = 0; v < V; ++v) {
                const float re = __builtin_fmaf(k[u].RhoPhiR, c[u][v], -(k[u].RhoPhiI * s[u][v]));
                const float im = __builtin_fmaf(k[u].RhoPhiI, c[u][v], k[u].RhoPhiR * s[u][v]);
                sOutR[v] += re;
                sOutI[v] += im;
            }
    }
    for (; kIndex < k_end; ++kIndex) {
        const mrif_kValues k = c_mrif[kIndex];
#pragma unroll
        for (int v = 0; v < V; ++v) {
            const float turn = __builtin_amdgcn_fractf(
                __builtin_fmaf(k.Kz, sZ[v], __builtin_fmaf(k.Ky, sY[v], k.Kx * sX[v])));
            const float c = __builtin_amdgcn_cosf(turn), s = __builtin_amdgcn_sinf(turn);
            sOutR[v] += __builtin_fmaf(k.RhoPhiR, c, -(k.RhoPhiI * s));
            sOutI[v] += __builtin_fmaf(k.RhoPhiI, c, k.RhoPhiR * s);
        }
    }
#pragma unroll
    for (int v = 0; v < V; ++v) {
        outR[xIndex[v]] = sOutR[v];
        outI[xIndex[v]] = sOutI[v];
    }
}

// the natural kernel's thread: one voxel, every record
__device__ __forceinline__ void mrif_voxel(int numK, const float *__restrict__ x,
                                           const float *__restrict__ y, const float *__restrict__ z,
                                           float *__restrict__ outR, float *__restrict__ outI, int xIndex)
{
    const int one[1] = {xIndex};
    mrif_voxels<1>(0, numK, x, y, z, outR, outI, one);
}

struct MrifBody {
    static __device__ __forceinline__ int chunk() { return MRIF_K_CHUNK; }
    template <int V>
    static __device__ __forceinline__ void voxels(int k_begin, int k_end, const float *__restrict__ x,
                                                  const float *__restrict__ y, const float *__restrict__ z,
                                                  float *__restrict__ outR, float *__restrict__ outI,
                                                  const int (&xIndex)[V])
    {
        mrif_voxels<V>(k_begin, k_end, x, y, z, outR, outI, xIndex);
    }
};

// Block positions [start, end) of the (voxel blocks) x (k chunks) grid, as mriq_role.
__device__ __forceinline__ void mrif_role(int numK, const float *__restrict__ x,
                                          const float *__restrict__ y, const float *__restrict__ z,
                                          float *__restrict__ outR, float *__restrict__ outI,
                                          int grid_dimension_x, int grid_dimension_y, int role_block,
                                          int role_blocks, int start, int end, int tid, int role_threads)
{
    mriq_role<MrifBody>(numK, x, y, z, outR, outI, grid_dimension_x, grid_dimension_y, role_block, role_blocks,
                        start, end, tid, role_threads);
}

}  // namespace tk
