// MRI-Q role: Q(x) += sum_k phiMag_k * exp(i 2 pi k.x).
//
// Replaces ori_mriq / g_general_ptb_mriq (src/ori_kernel/mriq_kernel.cu:56-105,
// src/gptb_kernel/mriq_kernel.cu:3-70).  The fused copy of the reference
// truncates cos/sin to int (src/mix_kernel/tzgemm_mriq.cu:57,63); parity is with
// the unfused kernel, so this role keeps float throughout.  Kept: one thread per
// voxel, blocks of 256 voxels, read-modify-write of Qr/Qi, the k table as an
// array of {Kx,Ky,Kz,PhiMag} in constant memory, fp32 order
//   arg = 2pi * ((Kx*x + Ky*y) + Kz*z); Qr += PhiMag*cos(arg); Qi += PhiMag*sin(arg)
// with k ascending.  The reference's loop "for QGrid < 1" handles only the first
// 1024-sample chunk; here the loop runs over all numK samples held in the table.
//
// gfx950: the table index is wave-uniform, so the compiler fetches each record
// with one scalar 16-byte load; the work is VALU/transcendental bound.
#pragma once
#include "role_common.h"
#include "../header/mriq_header.h"

__constant__ mriq_kValues ck[MRIQ_MAX_K];

namespace tk {

__device__ __forceinline__ void mriq_voxel(int numK, const float *__restrict__ x,
                                           const float *__restrict__ y, const float *__restrict__ z,
                                           float *__restrict__ Qr, float *__restrict__ Qi, int xIndex)
{
    const float sX = x[xIndex];
    const float sY = y[xIndex];
    const float sZ = z[xIndex];
    float sQr = Qr[xIndex];
    float sQi = Qi[xIndex];
    for (int kIndex = 0; kIndex < numK; ++kIndex) {
        const float expArg = PIx2_MRIQ * (ck[kIndex].Kx * sX + ck[kIndex].Ky * sY + ck[kIndex].Kz * sZ);
        float s, c;
        sincosf(expArg, &s, &c);
        sQr += ck[kIndex].PhiMag * c;
        sQi += ck[kIndex].PhiMag * s;
    }
    Qr[xIndex] = sQr;
    Qi[xIndex] = sQi;
}

__device__ __forceinline__ void mriq_role(int numK, const float *__restrict__ x,
                                          const float *__restrict__ y, const float *__restrict__ z,
                                          float *__restrict__ Qr, float *__restrict__ Qi,
                                          int grid_dimension_x, int role_block, int role_blocks,
                                          int start, int end, int tid, int role_threads)
{
    const int blocks_at_once = role_threads / KERNEL_Q_THREADS_PER_BLOCK;
    const int slot = tid / KERNEL_Q_THREADS_PER_BLOCK;
    const int t = tid % KERNEL_Q_THREADS_PER_BLOCK;
    if (slot >= blocks_at_once) return;
    const unsigned stride = (unsigned)role_blocks * blocks_at_once;
    for (unsigned pos = (unsigned)start + role_block * blocks_at_once + slot; pos < (unsigned)end;
         pos += stride) {
        const int bx = pos % grid_dimension_x;
        mriq_voxel(numK, x, y, z, Qr, Qi, bx * KERNEL_Q_THREADS_PER_BLOCK + t);
    }
}

}  // namespace tk
