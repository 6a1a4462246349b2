// hotspot3D role (Rodinia): one explicit time step of the heat equation on an nx x ny x nz chip,
// 7-point stencil plus the dissipated power, side faces insulated, top layer exchanging heat with
// the ambient.
//
// Replaces ori_hot3d / general_ptb_hot3d (src/ori_kernel/hot3d_kernel.cu:9-60,
// src/gptb_kernel/hot3d_kernel.cu:3-62 of the reference).  A block position is a
// block_dimension_x x block_dimension_y patch of columns (64 x 4 in the reference's launch); a
// thread owns one column (i, j) and marches it through the nz layers, bottom to top.  Per cell,
// in fp32 and in this order (no contraction):
//   out = cc*t + cw*W + ce*E + cs*S + cn*N + cb*below + ct*above + sdc*p + ct*80
// summed left to right, where W/E/N/S are the cell itself on the chip's edge, below is the cell
// itself in the bottom layer and above the cell itself in the top layer -- so the output is
// bit-identical to a CPU evaluation in the same order.
//
// gfx950: for the reference's 64 x 4 patch a wavefront serves a position -- a lane takes 4 adjacent
// columns of one row (16 lanes a row), so the next layer, the power and the rows to the north and
// south come as 16-byte loads and the step leaves as 16-byte stores; only the two values beyond
// the ends of the lane's four columns are single loads (from lines the wave fetched anyway).  The
// wavefronts of a workgroup take positions next to each other in x, which makes the workgroup's
// accesses 1 KiB runs per row.  Other patch shapes (and arrays that are not 16-byte aligned) take a
// column per lane.
#pragma once
#include "role_common.h"
#include "../header/hot3d_header.h"

namespace tk {

struct Hot3dCoefficients {
    float ce, cw, cn, cs, ct, cb, cc, sdc;
};

__device__ __forceinline__ float hot3d_cell(const Hot3dCoefficients &k, float centre, float w, float e, float s,
                                            float n, float below, float above, float power)
{
    return k.cc * centre + k.cw * w + k.ce * e + k.cs * s + k.cn * n + k.cb * below + k.ct * above +
           k.sdc * power + k.ct * HOT3D_AMB_TEMP;
}

// column (i, j), all layers
__device__ __forceinline__ void hot3d_column(const float *__restrict__ p, const float *__restrict__ tIn,
                                             float *__restrict__ tOut, const Hot3dCoefficients &k, int nx, int ny,
                                             int nz, int i, int j)
{
    const int xy = nx * ny;
    int c = i + j * nx;
    int W = (i == 0) ? c : c - 1;
    int E = (i == nx - 1) ? c : c + 1;
    int N = (j == 0) ? c : c - nx;
    int S = (j == ny - 1) ? c : c + nx;
    float below, centre, above;
    below = centre = tIn[c];
    above = tIn[c + xy];
    tOut[c] = hot3d_cell(k, centre, tIn[W], tIn[E], tIn[S], tIn[N], below, above, p[c]);
    c += xy, W += xy, E += xy, N += xy, S += xy;
#pragma unroll 2
    for (int layer = 1; layer < nz - 1; ++layer) {
        below = centre;
        centre = above;
        above = tIn[c + xy];
        tOut[c] = hot3d_cell(k, centre, tIn[W], tIn[E], tIn[S], tIn[N], below, above, p[c]);
        c += xy, W += xy, E += xy, N += xy, S += xy;
    }
    below = centre;
    centre = above;
    tOut[c] = hot3d_cell(k, centre, tIn[W], tIn[E], tIn[S], tIn[N], below, above, p[c]);
}

// the reference's 64 x 4 patch (bx, by) by one wavefront: lane -> row lane / 16, columns 4 (lane % 16) .. + 3
__device__ __forceinline__ void hot3d_patch_wave(const float *__restrict__ p, const float *__restrict__ tIn,
                                                 float *__restrict__ tOut, const Hot3dCoefficients &k, int nx, int ny,
                                                 int nz, int bx, int by, int lane)
{
    const int i = HOT3D_TILE_X * bx + 4 * (lane & 15);
    const int j = HOT3D_TILE_Y * by + (lane >> 4);
    if (i >= nx || j >= ny) return;
    const long long xy = (long long)nx * ny;
    long long c = i + (long long)j * nx;
    // offsets of the neighbours relative to c, the same in every layer
    const int w_off = (i == 0) ? 0 : -1;            // left of the first column
    const int e_off = (i + 3 == nx - 1) ? 3 : 4;    // right of the fourth
    const int n_off = (j == 0) ? 0 : -nx;
    const int s_off = (j == ny - 1) ? 0 : nx;
    float4 below, centre, above;
    below = centre = *reinterpret_cast<const float4 *>(tIn + c);
    for (int layer = 0; layer < nz; ++layer) {
        above = layer < nz - 1 ? *reinterpret_cast<const float4 *>(tIn + c + xy) : centre;
        const float4 north = *reinterpret_cast<const float4 *>(tIn + c + n_off);
        const float4 south = *reinterpret_cast<const float4 *>(tIn + c + s_off);
        const float4 power = *reinterpret_cast<const float4 *>(p + c);
        const float west = tIn[c + w_off], east = tIn[c + e_off];
        float4 out;
        out.x = hot3d_cell(k, centre.x, west, centre.y, south.x, north.x, below.x, above.x, power.x);
        out.y = hot3d_cell(k, centre.y, centre.x, centre.z, south.y, north.y, below.y, above.y, power.y);
        out.z = hot3d_cell(k, centre.z, centre.y, centre.w, south.z, north.z, below.z, above.z, power.z);
        out.w = hot3d_cell(k, centre.w, centre.z, east, south.w, north.w, below.w, above.w, power.w);
        *reinterpret_cast<float4 *>(tOut + c) = out;
        below = centre;
        centre = above;
        c += xy;
    }
}

// Block positions [start, end) of the grid (grid_dimension_x, grid_dimension_y) of patches of
// block_dimension_x x block_dimension_y columns are served by the role's role_blocks persistent
// workgroups in turn; positions wrap as the reference's block_pos % grid_dimension_x,
// (block_pos / grid_dimension_x) % grid_dimension_y do.  nz >= 2 (the reference reads the second
// layer unconditionally).
__device__ __forceinline__ void hot3d_role(const float *__restrict__ p, const float *__restrict__ tIn,
                                           float *__restrict__ tOut, float sdc, int nx, int ny, int nz, float ce,
                                           float cw, float cn, float cs, float ct, float cb, float cc,
                                           int grid_dimension_x, int grid_dimension_y, int block_dimension_x,
                                           int block_dimension_y, int role_block, int role_blocks, int start, int end,
                                           int tid, int role_threads)
{
    if (start >= end || grid_dimension_x <= 0 || grid_dimension_y <= 0 || block_dimension_x <= 0 ||
        block_dimension_y <= 0 || nz < 2)
        return;
    const Hot3dCoefficients k{ce, cw, cn, cs, ct, cb, cc, sdc};
    if (block_dimension_x == HOT3D_TILE_X && block_dimension_y == HOT3D_TILE_Y && nx % 4 == 0 &&
        (((size_t)p | (size_t)tIn | (size_t)tOut) & 15) == 0) {
        const int waves = role_threads / TK_WAVE_SIZE;
        const int wave = tid / TK_WAVE_SIZE;
        if (wave >= waves) return;
        const int lane = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
        // workgroup b takes positions (b + j role_blocks) waves + wave of the range, j = 0, 1, ...
        for (long long pos = (long long)start + (long long)role_block * waves + wave; pos < end;
             pos += (long long)role_blocks * waves) {
            const unsigned q = (unsigned)pos;
            hot3d_patch_wave(p, tIn, tOut, k, nx, ny, nz, (int)(q % (unsigned)grid_dimension_x),
                             (int)((q / (unsigned)grid_dimension_x) % (unsigned)grid_dimension_y), lane);
        }
        return;
    }
    const int patch = block_dimension_x * block_dimension_y;
    const int at_once = role_threads >= patch ? role_threads / patch : 1;
    const int group = role_threads >= patch ? tid / patch : 0;
    const int first = role_threads >= patch ? tid % patch : tid;
    const int step = role_threads >= patch ? patch : role_threads;
    if (group >= at_once) return;
    for (long long pos = (long long)start + role_block + (long long)group * role_blocks; pos < end;
         pos += (long long)at_once * role_blocks) {
        const unsigned q = (unsigned)pos;
        const int bx = (int)(q % (unsigned)grid_dimension_x);
        const int by = (int)((q / (unsigned)grid_dimension_x) % (unsigned)grid_dimension_y);
        for (int t = first; t < patch; t += step) {
            const int i = block_dimension_x * bx + t % block_dimension_x;
            const int j = block_dimension_y * by + t / block_dimension_x;
            if (i < nx && j < ny) hot3d_column(p, tIn, tOut, k, nx, ny, nz, i, j);
        }
    }
}

}  // namespace tk
