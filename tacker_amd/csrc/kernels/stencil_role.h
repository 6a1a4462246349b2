// 7-point Jacobi stencil role.
//
// Replaces ori_stencil / general_ptb_stencil / stencil_tzgemm_stencil0 of the
// reference (src/ori_kernel/stencil_kernel.cu:9-94, src/gptb_kernel/stencil_kernel.cu:3-104,
// src/mix_kernel/tzgemm_stencil.cu:174-277).  Kept: the block decomposition
// (block (bx,by) covers x in [64*bx, 64*bx+64), y in [4*by, 4*by+4), all z), the
// interior predicate, and the per-point operation order
//   Anext = (top + bottom + up + down + right + left)*c1 - centre*c0   (:68-69,:82-83)
// so that results are bit-identical to an ordered fp32 evaluation.
//
// gfx950 design: one wave64 per reference block, no LDS and no barrier.  Lane l
// owns column x = 64*bx + l and keeps ROWS rows of three consecutive z planes in
// registers (bottom / centre / top); y neighbours inside the block are the
// lane's own registers, x neighbours are the adjacent lanes' registers (wave
// shuffle), and only the halo (row above/below the block, column left/right of
// the wave) is read a second time, from L2.  Every global access of a wave is a
// contiguous 256-byte row segment.  Because a block needs no workgroup-level
// cooperation the role runs unchanged as a whole launch or as some waves of a
// fused workgroup.
#pragma once
#include "role_common.h"
#include "../header/stencil_header.h"

namespace tk {

// March one block column: x = x0 + lane, rows j0 .. j0+ROWS-1, k = 1 .. nz-2.
template <int ROWS>
__device__ __forceinline__ void stencil_wave_block(float c0, float c1, const float *__restrict__ A0,
                                                   float *__restrict__ Anext, int nx, int ny, int nz,
                                                   int x0, int j0, int lane)
{
    const int x = x0 + lane;
    const size_t plane = (size_t)nx * (size_t)ny;
    const bool xin = x < nx;
    const bool halo_dn = xin && j0 > 0;
    const bool halo_up = xin && (j0 + ROWS) < ny;
    // lane 0 fetches the column left of the wave, lane 63 the column right of it
    const bool edge_l = lane == 0 && x > 0 && xin;
    const bool edge_r = lane == 63 && (x + 1) < nx;
    const int edge_x = edge_l ? x - 1 : x + 1;

    float bot[ROWS], cur[ROWS], top[ROWS], edge[ROWS];
    float dn = 0.f, up = 0.f;
    bool rin[ROWS], win[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        const int j = j0 + r;
        rin[r] = xin && j < ny;
        win[r] = x > 0 && x < nx - 1 && j > 0 && j < ny - 1;
    }

    auto load_rows = [&](int k, float (&dst)[ROWS]) {
#pragma unroll
        for (int r = 0; r < ROWS; ++r)
            dst[r] = rin[r] ? A0[(size_t)x + (size_t)nx * (j0 + r) + plane * k] : 0.f;
    };
    auto load_halo = [&](int k, float &d, float &u, float (&e)[ROWS]) {
        d = halo_dn ? A0[(size_t)x + (size_t)nx * (j0 - 1) + plane * k] : 0.f;
        u = halo_up ? A0[(size_t)x + (size_t)nx * (j0 + ROWS) + plane * k] : 0.f;
#pragma unroll
        for (int r = 0; r < ROWS; ++r)
            e[r] = ((edge_l || edge_r) && (j0 + r) < ny)
                       ? A0[(size_t)edge_x + (size_t)nx * (j0 + r) + plane * k]
                       : 0.f;
    };

    load_rows(0, bot);
    load_rows(1, cur);
    load_halo(1, dn, up, edge);
    for (int k = 1; k < nz - 1; ++k) {
        float ndn, nup, nedge[ROWS];
        load_rows(k + 1, top);
        load_halo(k + 1, ndn, nup, nedge);   // neighbours of the next centre plane
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            float left = __shfl_up(cur[r], 1, 64);
            float right = __shfl_down(cur[r], 1, 64);
            if (lane == 0) left = edge[r];
            if (lane == 63) right = edge[r];
            const float a_up = (r + 1 < ROWS) ? cur[(r + 1 < ROWS) ? r + 1 : r] : up;
            const float a_dn = (r > 0) ? cur[(r > 0) ? r - 1 : r] : dn;
            if (win[r]) {
                float s = top[r] + bot[r];
                s = s + a_up;
                s = s + a_dn;
                s = s + right;
                s = s + left;
                Anext[(size_t)x + (size_t)nx * (j0 + r) + plane * k] = s * c1 - cur[r] * c0;
            }
        }
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            bot[r] = cur[r];
            cur[r] = top[r];
            edge[r] = nedge[r];
        }
        dn = ndn;
        up = nup;
    }
}

// GPTB form: virtual block = one wave.  The role's waves enumerate block
// positions start + (role_block*waves + wave) + i*(role_blocks*waves).
__device__ __forceinline__ void stencil_role(float c0, float c1, const float *__restrict__ A0,
                                             float *__restrict__ Anext, int nx, int ny, int nz,
                                             int grid_dimension_x, int grid_dimension_y,
                                             int role_block, int role_blocks, int start, int end,
                                             int tid, int role_threads)
{
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int waves = role_threads >> 6;
    const unsigned stride = (unsigned)role_blocks * waves;
    for (unsigned pos = (unsigned)start + role_block * waves + wave; pos < (unsigned)end;
         pos += stride) {
        const int bx = pos % grid_dimension_x;
        const int by = (pos / grid_dimension_x) % grid_dimension_y;
        stencil_wave_block<STENCIL_TILE_Y>(c0, c1, A0, Anext, nx, ny, nz, bx * 2 * STENCIL_TILE_X,
                                           by * STENCIL_TILE_Y, lane);
    }
}

}  // namespace tk
