// Coulomb-potential role: one z slice of the potential of up to 64 point charges.
//
// Replaces ori_cp / g_general_ptb_cp / cp_tzgemm_cp0 (src/ori_kernel/cp_kernel.cu:26-79,
// src/gptb_kernel/cp_kernel.cu:8-96, src/mix_kernel/tzgemm_cp.cu:6-94).  Kept
// verbatim in meaning: (16,8) thread blocks, 8 x-points per thread 16 apart,
// atoms {x, y, dz^2, q} in constant memory, and the fp32 operation order
//   dy = coory - a.y; dyz2 = dy*dy + a.z; dx_{n+1} = dx_n + 16*spacing;
//   E_n += a.w * (1.0f / sqrtf(dx_n*dx_n + dyz2)); energygrid[...] += E_n
// so the output is bit-identical to a CPU evaluation with IEEE sqrt and divide.
//
// gfx950: 16 lanes write 64 contiguous bytes and the 8 unrolled points of a row
// tile a contiguous 512-byte span; atoms are read with scalar loads.
#pragma once
#include "role_common.h"
#include "../header/cp_header.h"

__constant__ float4 atominfo[MAXATOMS];

namespace tk {

__device__ __forceinline__ void cp_block(int numatoms, float gridspacing,
                                         float *__restrict__ energygrid, unsigned block_id_x,
                                         unsigned block_id_y, unsigned grid_dimension_x,
                                         unsigned thread_id_x, unsigned thread_id_y)
{
    const unsigned xindex = block_id_x * BLOCKSIZEX * UNROLLX + thread_id_x;
    const unsigned yindex = block_id_y * BLOCKSIZEY + thread_id_y;
    const unsigned outaddr = (grid_dimension_x * BLOCKSIZEX * UNROLLX) * yindex + xindex;

    const float coory = gridspacing * yindex;
    const float coorx = gridspacing * xindex;
    float energyval[UNROLLX];
#pragma unroll
    for (int n = 0; n < UNROLLX; ++n) energyval[n] = 0.0f;
    const float gridspacing_u = gridspacing * BLOCKSIZEX;

    for (int atomid = 0; atomid < numatoms; ++atomid) {
        const float dy = coory - atominfo[atomid].y;
        const float dyz2 = (dy * dy) + atominfo[atomid].z;
        float dx = coorx - atominfo[atomid].x;
#pragma unroll
        for (int n = 0; n < UNROLLX; ++n) {
            energyval[n] += atominfo[atomid].w * (1.0f / sqrtf(dx * dx + dyz2));
            dx = dx + gridspacing_u;
        }
    }
#pragma unroll
    for (int n = 0; n < UNROLLX; ++n) energygrid[outaddr + n * BLOCKSIZEX] += energyval[n];
}

// Two blocks per thread at once: 16 independent sqrt/divide chains instead of 8.  A fused
// launch leaves this role two waves per SIMD; with one block per thread the IEEE sqrt and
// divide sequences (each a dependent chain of about ten instructions) do not fill the VALU.
// Every output keeps its own chain in the order of cp_block, so values are unchanged.
__device__ __forceinline__ void cp_block_pair(int numatoms, float gridspacing,
                                              float *__restrict__ energygrid, const unsigned (&bx)[2],
                                              const unsigned (&by)[2], unsigned grid_dimension_x,
                                              unsigned thread_id_x, unsigned thread_id_y)
{
    unsigned outaddr[2];
    float coory[2], coorx[2];
    float energyval[2][UNROLLX];
#pragma unroll
    for (int b = 0; b < 2; ++b) {
        const unsigned xindex = bx[b] * BLOCKSIZEX * UNROLLX + thread_id_x;
        const unsigned yindex = by[b] * BLOCKSIZEY + thread_id_y;
        outaddr[b] = (grid_dimension_x * BLOCKSIZEX * UNROLLX) * yindex + xindex;
        coory[b] = gridspacing * yindex;
        coorx[b] = gridspacing * xindex;
#pragma unroll
        for (int n = 0; n < UNROLLX; ++n) energyval[b][n] = 0.0f;
    }
    const float gridspacing_u = gridspacing * BLOCKSIZEX;
    for (int atomid = 0; atomid < numatoms; ++atomid) {
        const float4 a = atominfo[atomid];
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            const float dy = coory[b] - a.y;
            const float dyz2 = (dy * dy) + a.z;
            float dx = coorx[b] - a.x;
#pragma unroll
            for (int n = 0; n < UNROLLX; ++n) {
                energyval[b][n] += a.w * (1.0f / sqrtf(dx * dx + dyz2));
                dx = dx + gridspacing_u;
            }
        }
    }
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int n = 0; n < UNROLLX; ++n) energygrid[outaddr[b] + n * BLOCKSIZEX] += energyval[b][n];
}

__device__ __forceinline__ void cp_role(int numatoms, float gridspacing,
                                        float *__restrict__ energygrid, int grid_dimension_x,
                                        int grid_dimension_y, int role_block, int role_blocks,
                                        int start, int end, int tid, int role_threads)
{
    constexpr int BLOCK_THREADS = BLOCKSIZEX * BLOCKSIZEY;
    const int blocks_at_once = role_threads / BLOCK_THREADS;
    const int slot = tid / BLOCK_THREADS;
    const int t = tid % BLOCK_THREADS;
    if (slot >= blocks_at_once) return;
    const unsigned stride = (unsigned)role_blocks * blocks_at_once;
    // blocks go round the role's workgroups first; a thread takes two that are one stride apart
    // (two positions of one launch never name the same block unless the range wraps, and a
    // wrapped range is served one block at a time so that its += land one after the other)
    const bool wraps = (unsigned)(end - start) > (unsigned)(grid_dimension_x * grid_dimension_y);
    for (unsigned pos = (unsigned)start + slot * role_blocks + role_block; pos < (unsigned)end;
         pos += 2 * stride) {
        const unsigned second = pos + stride;
        if (second < (unsigned)end && !wraps) {
            const unsigned bx[2] = {pos % grid_dimension_x, second % grid_dimension_x};
            const unsigned by[2] = {(pos / grid_dimension_x) % grid_dimension_y,
                                    (second / grid_dimension_x) % grid_dimension_y};
            cp_block_pair(numatoms, gridspacing, energygrid, bx, by, grid_dimension_x, t % BLOCKSIZEX,
                          t / BLOCKSIZEX);
        } else {
            cp_block(numatoms, gridspacing, energygrid, pos % grid_dimension_x,
                     (pos / grid_dimension_x) % grid_dimension_y, grid_dimension_x, t % BLOCKSIZEX,
                     t / BLOCKSIZEX);
            if (second < (unsigned)end)
                cp_block(numatoms, gridspacing, energygrid, second % grid_dimension_x,
                         (second / grid_dimension_x) % grid_dimension_y, grid_dimension_x,
                         t % BLOCKSIZEX, t / BLOCKSIZEX);
        }
    }
}

}  // namespace tk
