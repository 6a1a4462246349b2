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
// registers.  The neighbours across lanes come by lane shuffles, so the two block barriers a row
// of the reference's block and its two shared arrays are gone; the rows of the wall, the only
// memory traffic, are fetched PATH_ROWS_AHEAD rows ahead of the row being evaluated (the
// dynamic programme itself is a dependent chain of `iteration` steps).
#pragma once
#include "role_common.h"
#include "../header/path_header.h"

#define PATH_ROWS_AHEAD 8

namespace tk {

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

    int prev[C], result[C];
    bool valid[C];
#pragma unroll
    for (int k = 0; k < C; ++k) {
        const int tx = tx0 + k, xidx = blkX + tx;
        valid[k] = tx >= validXmin && tx <= validXmax;
        prev[k] = (xidx >= 0 && xidx <= cols - 1) ? gpuSrc[xidx] : 0;
        result[k] = 0;
    }
    // row i of the wall for this lane's columns, where they take part in row i
    auto fetch = [&](int i, int (&w)[C]) {
        const long long row = (long long)cols * (startStep + i) + blkX;
#pragma unroll
        for (int k = 0; k < C; ++k) {
            const int tx = tx0 + k;
            const bool takes_part = i < iteration && valid[k] && tx >= i + 1 && tx <= PATH_BLOCK_SIZE - i - 2;
            w[k] = takes_part ? gpuWall[row + tx] : 0;
        }
    };
    int wall[PATH_ROWS_AHEAD][C];
#pragma unroll
    for (int u = 0; u < PATH_ROWS_AHEAD; ++u) fetch(u, wall[u]);

    bool computed[C];
#pragma unroll
    for (int k = 0; k < C; ++k) computed[k] = false;
    for (int base = 0; base < iteration; base += PATH_ROWS_AHEAD) {
#pragma unroll
        for (int u = 0; u < PATH_ROWS_AHEAD; ++u) {
            const int i = base + u;
            if (i >= iteration) break;   // uniform
            // the columns next to this lane's four
            const int from_left = __shfl_up(prev[C - 1], 1);
            const int from_right = __shfl_down(prev[0], 1);
#pragma unroll
            for (int k = 0; k < C; ++k) {
                const int tx = tx0 + k;
                computed[k] = valid[k] && tx >= i + 1 && tx <= PATH_BLOCK_SIZE - i - 2;
                const int left_of = k == 0 ? from_left : prev[k - 1];
                const int right_of = k == C - 1 ? from_right : prev[k + 1];
                const int left = tx == validXmin ? prev[k] : left_of;      // W clamped to validXmin
                const int right = tx == validXmax ? prev[k] : right_of;    // E clamped to validXmax
                const int up = prev[k];
                int shortest = left <= up ? left : up;
                shortest = shortest <= right ? shortest : right;
                if (computed[k]) result[k] = shortest + wall[u][k];
            }
            if (i == iteration - 1) break;   // uniform
#pragma unroll
            for (int k = 0; k < C; ++k)
                if (computed[k]) prev[k] = result[k];
            fetch(i + PATH_ROWS_AHEAD, wall[u]);
        }
    }
#pragma unroll
    for (int k = 0; k < C; ++k)
        if (computed[k]) gpuResults[blkX + tx0 + k] = result[k];
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
