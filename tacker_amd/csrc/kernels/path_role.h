// pathfinder role (Rodinia): `iteration` rows of the dynamic programme
//   next[x] = wall[row][x] + min(prev[x-1], prev[x], prev[x+1])      (x clamped to the grid)
// evaluated block by block on overlapping 256-column windows (a pyramid: every row the window's
// computed part shrinks by one column on each side, and the PATH_BLOCK_SIZE - 2 * iteration
// columns left in the middle are the block's result).
//
// Replaces ori_path / general_ptb_path (src/ori_kernel/path_kernel.cu:9-86,
// src/gptb_kernel/path_kernel.cu:3-93 of the reference).  Integer work: the output is the
// reference's bit for bit.  A block position bx is the window of columns
//   [small * bx - border, small * bx - border + 255],   small = 256 - 2 * iteration,
// column tx of it takes part in row i when i + 1 <= tx <= 254 - i and the column lies on the grid,
// with the neighbours clamped to the window's columns on the grid; after the last row the columns
// that were computed in it are written to gpuResults.
//
// gfx950: a wavefront serves a position, a lane holds 4 consecutive columns of the window in
// registers.  The neighbours across lanes come by a one-lane DPP shift of the wavefront, so the two
// block barriers a row of the reference's block and its two shared arrays are gone.  The dynamic
// programme is a dependent chain of `iteration` steps issued by one wavefront, so a step is kept to
// a few instructions: every column is updated in every row without asking whether it still takes
// part -- a column outside the shrinking pyramid holds a value nobody reads, since a column that
// takes part in row i only reads columns that took part in row i - 1 -- and only the clamping at
// the grid's two edges and the final store are predicated.  The rows of the wall, the only memory
// traffic, are fetched PATH_ROWS_AHEAD rows ahead of the row being evaluated, from column indices
// clamped to the grid so that no load needs a predicate either.
#pragma once
#include "role_common.h"
#include "../header/path_header.h"

#ifndef PATH_ROWS_AHEAD
#define PATH_ROWS_AHEAD 8
#endif

namespace tk {

// value of the lane below / above in the wavefront (the lane itself at the wavefront's ends)
__device__ __forceinline__ int path_from_lane_below(int v)
{
    return __builtin_amdgcn_update_dpp(v, v, 0x138 /* wave_shr:1 */, 0xf, 0xf, false);
}
__device__ __forceinline__ int path_from_lane_above(int v)
{
    return __builtin_amdgcn_update_dpp(v, v, 0x130 /* wave_shl:1 */, 0xf, 0xf, false);
}

// one position, whole pyramid; lane = lane of the wavefront
__device__ __forceinline__ void path_window(int iteration, const int *__restrict__ gpuWall,
                                            const int *__restrict__ gpuSrc, int *__restrict__ gpuResults, int cols,
                                            int startStep, int border, int bx, int lane)
{
    constexpr int C = PATH_COLS_PER_LANE;
    const int small_block_cols = PATH_BLOCK_SIZE - iteration * PATH_HALO * 2;
    const int blkX = small_block_cols * bx - border;
    const int blkXmax = blkX + PATH_BLOCK_SIZE - 1;
    const int validXmin = (blkX < 0) ? -blkX : 0;
    const int validXmax = (blkXmax > cols - 1) ? PATH_BLOCK_SIZE - 1 - (blkXmax - cols + 1) : PATH_BLOCK_SIZE - 1;
    const int tx0 = C * lane;

    int prev[C];
    unsigned column[C];   // unsigned: a load is a wave-uniform row pointer plus a 32-bit lane offset
    bool at_min[C], at_max[C];
#pragma unroll
    for (int k = 0; k < C; ++k) {
        const int tx = tx0 + k, xidx = blkX + tx;
        column[k] = (unsigned)(xidx < 0 ? 0 : (xidx > cols - 1 ? cols - 1 : xidx));   // on the grid, for the loads
        at_min[k] = tx == validXmin;                                       // W clamps to the column itself
        at_max[k] = tx == validXmax;                                       // E likewise
        prev[k] = gpuSrc[column[k]];
    }
    const int *ahead = gpuWall + (long long)cols * startStep;   // the row the next fetch takes
    int wall[PATH_ROWS_AHEAD][C];
#pragma unroll
    for (int u = 0; u < PATH_ROWS_AHEAD; ++u)
        if (u < iteration) {
#pragma unroll
            for (int k = 0; k < C; ++k) wall[u][k] = ahead[column[k]];
            ahead += cols;
        }
    for (int base = 0; base < iteration; base += PATH_ROWS_AHEAD) {
#pragma unroll
        for (int u = 0; u < PATH_ROWS_AHEAD; ++u) {
            const int i = base + u;
            if (i >= iteration) break;   // uniform
            const int from_left = path_from_lane_below(prev[C - 1]);
            const int from_right = path_from_lane_above(prev[0]);
            int next[C];
#pragma unroll
            for (int k = 0; k < C; ++k) {
                const int left = at_min[k] ? prev[k] : (k == 0 ? from_left : prev[k - 1]);
                const int right = at_max[k] ? prev[k] : (k == C - 1 ? from_right : prev[k + 1]);
                int shortest = left <= prev[k] ? left : prev[k];
                shortest = shortest <= right ? shortest : right;
                next[k] = shortest + wall[u][k];
            }
#pragma unroll
            for (int k = 0; k < C; ++k) prev[k] = next[k];
            if (i + PATH_ROWS_AHEAD < iteration) {   // uniform
#pragma unroll
                for (int k = 0; k < C; ++k) wall[u][k] = ahead[column[k]];
                ahead += cols;
            }
        }
    }
    // the columns that took part in the last row: the middle of the window, where it is on the grid
#pragma unroll
    for (int k = 0; k < C; ++k) {
        const int tx = tx0 + k;
        if (tx >= iteration && tx <= PATH_BLOCK_SIZE - 1 - iteration && tx >= validXmin && tx <= validXmax)
            gpuResults[blkX + tx] = prev[k];
    }
}

// Block positions [start, end) are served by the role's role_blocks x (role_threads / 64)
// wavefronts in turn; the position is the reference's bx (it uses block_pos itself, no wrap).
__device__ __forceinline__ void path_role(int iteration, const int *__restrict__ gpuWall,
                                          const int *__restrict__ gpuSrc, int *__restrict__ gpuResults, int cols,
                                          int startStep, int border, int role_block, int role_blocks, int start,
                                          int end, int tid, int role_threads)
{
    const int waves = role_threads / TK_WAVE_SIZE;
    const int wave = tid / TK_WAVE_SIZE;
    if (wave >= waves || start >= end || iteration <= 0 || 2 * iteration >= PATH_BLOCK_SIZE) return;
    const int lane = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    for (long long pos = (long long)start + role_block + (long long)role_blocks * wave; pos < end;
         pos += (long long)role_blocks * waves)
        path_window(iteration, gpuWall, gpuSrc, gpuResults, cols, startStep, border, (int)pos, lane);
}

}  // namespace tk
