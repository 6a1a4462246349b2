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
// with one scalar 16-byte load; the work is VALU/transcendental bound.  The
// hardware sine and cosine take their argument in revolutions, so the phase
// k.x is used as it is (reduced with v_fract) instead of being scaled by 2 pi
// and reduced again in software: cos(2 pi p) = v_cos(fract(p)).  The dot product
// keeps the reference's order and separate roundings; the result differs from a
// float64 evaluation by about 1e-6 per term, far inside the 1e-3 + 1e-4 |Q| bar.
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
#pragma unroll 8
    for (int kIndex = 0; kIndex < numK; ++kIndex) {
        const float phase = ck[kIndex].Kx * sX + ck[kIndex].Ky * sY + ck[kIndex].Kz * sZ;   // revolutions
        const float turn = __builtin_amdgcn_fractf(phase);
        const float s = __builtin_amdgcn_sinf(turn);
        const float c = __builtin_amdgcn_cosf(turn);
        sQr += ck[kIndex].PhiMag * c;
        sQi += ck[kIndex].PhiMag * s;
    }
    Qr[xIndex] = sQr;
    Qi[xIndex] = sQi;
}

// V voxels per thread at once.  The k loop is a chain of dependent operations per voxel
// (dot product, fract, sin/cos, accumulate) and a fused launch leaves the role at most two
// waves per SIMD, so the independent work that hides instruction latency has to come
// from inside the thread; V voxels also share each scalar load of a k record.
template <int V>
__device__ __forceinline__ void mriq_voxels(int numK, const float *__restrict__ x,
                                            const float *__restrict__ y, const float *__restrict__ z,
                                            float *__restrict__ Qr, float *__restrict__ Qi,
                                            const int (&xIndex)[V], int count)
{
    float sX[V], sY[V], sZ[V], sQr[V], sQi[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
        const int i = xIndex[v < count ? v : 0];
        sX[v] = x[i];
        sY[v] = y[i];
        sZ[v] = z[i];
        sQr[v] = Qr[i];
        sQi[v] = Qi[i];
    }
    // unrolled so the scalar loads of 8 records are issued together: one record per
    // iteration would put a scalar-cache round trip on every step of the chain
#pragma unroll 8
    for (int kIndex = 0; kIndex < numK; ++kIndex) {
        const mriq_kValues k = ck[kIndex];
#pragma unroll
        for (int v = 0; v < V; ++v) {
            const float phase = k.Kx * sX[v] + k.Ky * sY[v] + k.Kz * sZ[v];   // revolutions
            const float turn = __builtin_amdgcn_fractf(phase);
            sQr[v] += k.PhiMag * __builtin_amdgcn_cosf(turn);
            sQi[v] += k.PhiMag * __builtin_amdgcn_sinf(turn);
        }
    }
#pragma unroll
    for (int v = 0; v < V; ++v)
        if (v < count) {
            Qr[xIndex[v]] = sQr[v];
            Qi[xIndex[v]] = sQi[v];
        }
}

#define MRIQ_VOXELS_PER_THREAD 4
__device__ __forceinline__ void mriq_role(int numK, const float *__restrict__ x,
                                          const float *__restrict__ y, const float *__restrict__ z,
                                          float *__restrict__ Qr, float *__restrict__ Qi,
                                          int grid_dimension_x, int role_block, int role_blocks,
                                          int start, int end, int tid, int role_threads)
{
    constexpr int V = MRIQ_VOXELS_PER_THREAD;
    const int blocks_at_once = role_threads / KERNEL_Q_THREADS_PER_BLOCK;
    const int slot = tid / KERNEL_Q_THREADS_PER_BLOCK;
    const int t = tid % KERNEL_Q_THREADS_PER_BLOCK;
    if (slot >= blocks_at_once) return;
    // block slots go round the role's workgroups first (slot-major), so a short range
    // still spreads over all CUs; a thread takes V blocks that are one stride apart
    const unsigned stride = (unsigned)role_blocks * blocks_at_once;
    for (unsigned pos = (unsigned)start + slot * role_blocks + role_block; pos < (unsigned)end;
         pos += stride * V) {
        int idx[V];
        int count = 0;
#pragma unroll
        for (int v = 0; v < V; ++v) {
            const unsigned p = pos + v * stride;
            idx[v] = (int)(p % grid_dimension_x) * KERNEL_Q_THREADS_PER_BLOCK + t;
            if (p < (unsigned)end) count = v + 1;
        }
        if (count > 2) {
            mriq_voxels<V>(numK, x, y, z, Qr, Qi, idx, count);
        } else if (count == 2) {
            const int two[2] = {idx[0], idx[1]};
            mriq_voxels<2>(numK, x, y, z, Qr, Qi, two, 2);
        } else {
            mriq_voxel(numK, x, y, z, Qr, Qi, idx[0]);
        }
    }
}

}  // namespace tk
