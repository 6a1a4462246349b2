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
// 1024-sample chunk; here all numK samples held in the table are used.
//
// gfx950: the table index is wave-uniform, so the compiler fetches each record
// with one scalar 16-byte load; the work is VALU/transcendental bound.  The
// hardware sine and cosine take their argument in revolutions, so the phase
// k.x is used as it is (reduced with v_fract) instead of being scaled by 2 pi
// and reduced again in software: cos(2 pi p) = v_cos(fract(p)).  The dot product and
// the two accumulations are fused multiply-adds in the reference's order
// (((Kx*x) + Ky*y) + Kz*z; Q + PhiMag*c) -- what nvcc makes of the reference's source
// with its default -fmad=true -- 8 instructions per (k, x) pair instead of 13.  The
// result differs from a float64 evaluation by about 1e-6 per term, far inside the
// 1e-3 + 1e-4 |Q| bar.
#pragma once
#include "role_common.h"
#include "../header/mriq_header.h"

__constant__ mriq_kValues ck[MRIQ_MAX_K];

namespace tk {

// V voxels per thread at once, k records [k_begin, k_end).  The k loop is a chain of
// dependent operations per voxel (dot product, fract, sin/cos, accumulate) and a fused
// launch leaves the role at most two waves per SIMD, so the independent work that hides
// instruction latency has to come from inside the thread; V voxels also share each
// scalar load of a k record.
template <int V>
__device__ __forceinline__ void mriq_voxels(int k_begin, int k_end, const float *__restrict__ x,
                                            const float *__restrict__ y, const float *__restrict__ z,
                                            float *__restrict__ Qr, float *__restrict__ Qi,
                                            const int (&xIndex)[V])
{
    float sX[V], sY[V], sZ[V], sQr[V], sQi[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
        const int i = xIndex[v];
        sX[v] = x[i];
        sY[v] = y[i];
        sZ[v] = z[i];
        sQr[v] = Qr[i];
        sQi[v] = Qi[i];
    }
    // U records at a time, written stage by stage (all phases, then all sines and cosines,
    // then the accumulation in ascending k): the U * V chains are independent until the last
    // stage, and the order of the source is already the interleaved one -- the compiler's
    // scheduler does not have to find it (for one of the instances in a fused kernel it did
    // not, and that loop ran one dependent chain at a time).  The scalar loads of the U
    // records are issued together: one record per iteration would put a scalar-cache round
    // trip on every step.
    constexpr int U = V >= 4 ? 4 : 8;
    int kIndex = k_begin;
    for (; kIndex + U <= k_end; kIndex += U) {
        mriq_kValues k[U];
#pragma unroll
        for (int u = 0; u < U; ++u) k[u] = ck[kIndex + u];
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
                sQr[v] = __builtin_fmaf(k[u].PhiMag, c[u][v], sQr[v]);
                sQi[v] = __builtin_fmaf(k[u].PhiMag, s[u][v], sQi[v]);
            }
    }
    for (; kIndex < k_end; ++kIndex) {
        const mriq_kValues k = ck[kIndex];
#pragma unroll
        for (int v = 0; v < V; ++v) {
            const float turn = __builtin_amdgcn_fractf(
                __builtin_fmaf(k.Kz, sZ[v], __builtin_fmaf(k.Ky, sY[v], k.Kx * sX[v])));
            sQr[v] = __builtin_fmaf(k.PhiMag, __builtin_amdgcn_cosf(turn), sQr[v]);
            sQi[v] = __builtin_fmaf(k.PhiMag, __builtin_amdgcn_sinf(turn), sQi[v]);
        }
    }
#pragma unroll
    for (int v = 0; v < V; ++v) {
        Qr[xIndex[v]] = sQr[v];
        Qi[xIndex[v]] = sQi[v];
    }
}

// the natural kernel's thread: one voxel, every record
__device__ __forceinline__ void mriq_voxel(int numK, const float *__restrict__ x,
                                           const float *__restrict__ y, const float *__restrict__ z,
                                           float *__restrict__ Qr, float *__restrict__ Qi, int xIndex)
{
    const int one[1] = {xIndex};
    mriq_voxels<1>(0, numK, x, y, z, Qr, Qi, one);
}

// What a thread does for V voxels and a run of k records: the part of the kernel that the
// walk over block positions below does not know about.  MRI-FHD (mrif_role.h) walks the
// same position grid with another body.
struct MriqBody {
    static __device__ __forceinline__ int chunk() { return MRIQ_K_CHUNK; }
    template <int V>
    static __device__ __forceinline__ void voxels(int k_begin, int k_end, const float *__restrict__ x,
                                                  const float *__restrict__ y, const float *__restrict__ z,
                                                  float *__restrict__ Qr, float *__restrict__ Qi,
                                                  const int (&xIndex)[V])
    {
        mriq_voxels<V>(k_begin, k_end, x, y, z, Qr, Qi, xIndex);
    }
};

// One phase of a launch: voxel blocks [block_lo, block_hi) each take records
// [k_begin, k_end).  A thread serves the blocks it owns -- first_owned, first_owned +
// stride, ... -- up to MRIQ_VOXELS_PER_THREAD at a time.
#define MRIQ_VOXELS_PER_THREAD 4
template <class Body>
__device__ __forceinline__ void mriq_phase(int block_lo, int block_hi, int k_begin, int k_end,
                                           const float *__restrict__ x, const float *__restrict__ y,
                                           const float *__restrict__ z, float *__restrict__ Qr,
                                           float *__restrict__ Qi, int first_owned, int stride, int t)
{
    constexpr int V = MRIQ_VOXELS_PER_THREAD;
    if (block_lo >= block_hi || k_begin >= k_end) return;
    int b = first_owned;
    if (b < block_lo) b += (block_lo - b + stride - 1) / stride * stride;
    for (; b < block_hi; b += V * stride) {
        int idx[V];
        int count = 0;
#pragma unroll
        for (int v = 0; v < V; ++v) {
            const int bv = b + v * stride;
            if (bv < block_hi) count = v + 1;
            idx[v] = (bv < block_hi ? bv : b) * KERNEL_Q_THREADS_PER_BLOCK + t;
        }
        if (count == V) {
            Body::template voxels<V>(k_begin, k_end, x, y, z, Qr, Qi, idx);
        } else {
            if (count >= 2) {
                const int two[2] = {idx[0], idx[1]};
                Body::template voxels<2>(k_begin, k_end, x, y, z, Qr, Qi, two);
            }
            if (count & 1) {
                const int one[1] = {idx[count - 1]};
                Body::template voxels<1>(k_begin, k_end, x, y, z, Qr, Qi, one);
            }
        }
    }
}

// Block positions of the GPTB form are a grid of grid_dimension_x voxel blocks (256 voxels
// each) by grid_dimension_y chunks of MRIQ_K_CHUNK k records: position p adds chunk
// (p / grid_dimension_x) % grid_dimension_y to voxel block p % grid_dimension_x -- the
// reference's host loop over k chunks (one launch per chunk with kGlobalIndex,
// src/ori_kernel/mriq_kernel.cu:258-283) folded into the y index of the GPTB grid, so that
// a short range of positions is a short piece of work.  Q is carried through memory
// between chunks exactly as the reference carries it between launches, and a float stored
// and reloaded is unchanged, so any split of [0, x*y) into ranges gives the bits of the
// one k loop.
//
// A range [start, end) is a partial first row of the position grid, whole rows, and a
// partial last row.  Every voxel block has one owner thread group for the whole launch
// (slot-major over the role's workgroups, so a short range still spreads over all CUs),
// and the owner walks the three parts in order: the chunks of a voxel are added in
// ascending position order without any synchronisation between threads.  Whole rows that
// follow each other are one run of the k loop.
template <class Body = MriqBody>
__device__ __forceinline__ void mriq_role(int numK, const float *__restrict__ x,
                                          const float *__restrict__ y, const float *__restrict__ z,
                                          float *__restrict__ Qr, float *__restrict__ Qi,
                                          int grid_dimension_x, int grid_dimension_y, int role_block,
                                          int role_blocks, int start, int end, int tid, int role_threads)
{
    const int blocks_at_once = role_threads / KERNEL_Q_THREADS_PER_BLOCK;
    const int slot = tid / KERNEL_Q_THREADS_PER_BLOCK;
    const int t = tid % KERNEL_Q_THREADS_PER_BLOCK;
    if (slot >= blocks_at_once || start >= end) return;
    const int gx = grid_dimension_x;
    const int gy = grid_dimension_y;
    const int stride = role_blocks * blocks_at_once;
    const int first_owned = slot * role_blocks + role_block;
    const auto chunk_begin = [&](int row) { return min((row % gy) * Body::chunk(), numK); };
    const auto chunk_end = [&](int row) { return min((row % gy + 1) * Body::chunk(), numK); };

    const int first_row = start / gx;
    const int last_row = (end - 1) / gx;   // row of the last position
    if (first_row == last_row) {
        mriq_phase<Body>(start - first_row * gx, end - first_row * gx, chunk_begin(first_row), chunk_end(first_row),
                   x, y, z, Qr, Qi, first_owned, stride, t);
        return;
    }
    int row = first_row;
    if (start != first_row * gx) {   // partial first row
        mriq_phase<Body>(start - first_row * gx, gx, chunk_begin(row), chunk_end(row), x, y, z, Qr, Qi,
                   first_owned, stride, t);
        ++row;
    }
    const int whole_end = (end == (last_row + 1) * gx) ? last_row + 1 : last_row;   // whole rows [row, whole_end)
    while (row < whole_end) {
        // rows up to the next multiple of grid_dimension_y are consecutive chunks
        const int run_end = min(whole_end, (row / gy + 1) * gy);
        mriq_phase<Body>(0, gx, chunk_begin(row), chunk_end(run_end - 1), x, y, z, Qr, Qi, first_owned, stride, t);
        row = run_end;
    }
    if (whole_end == last_row)       // partial last row
        mriq_phase<Body>(0, end - last_row * gx, chunk_begin(last_row), chunk_end(last_row), x, y, z, Qr, Qi,
                   first_owned, stride, t);
}

}  // namespace tk
