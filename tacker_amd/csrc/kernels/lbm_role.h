// D3Q19 lattice-Boltzmann role (collide + scatter, one time step).
//
// Replaces ori_lbm / general_ptb_lbm / lbm_tzgemm_lbm0 of the reference
// (src/ori_kernel/lbm_kernel.cu:9-154, src/gptb_kernel/lbm_kernel.cu:3-178,
// src/mix_kernel/tzgemm_lbm.cu:6-181) with run-time grid extents.  Kept: SoA
// layout CALC_INDEX(x,y,z,e) = cells*e + x + y*sx + z*sx*sy, SCATTER streaming
// by linear index arithmetic without boundary clamping, obstacle bounce-back,
// ACCEL override, and the exact fp32 operation order of the collision.
//
// One departure, on purpose: a scatter whose linear target cell lies outside
// [0, cells) would land in the neighbouring entry plane, where the reference
// races with that plane's own writer.  Here such a store is dropped, i.e. the
// race is always resolved in favour of the in-range writer, so results are
// reproducible.
//
// gfx950 design: a block is one x-row (y,z); a lane takes two x-adjacent cells (one
// if the row length is odd), so each of the 20 loads and 19 stores of a wave is one
// contiguous row segment of 8 bytes per lane.  No LDS, no barrier.
// A role of T threads processes T / roundup64(lanes per row) rows at once.
#pragma once
#include "role_common.h"
#include "../header/lbm_header.h"

namespace tk {

// All indices are 32-bit: the host refuses grids with 20*cells >= 2^31.

// Collision of one cell, in place (src/ori_kernel/lbm_kernel.cu:49-131): obstacle cells
// swap opposite directions, the others relax towards equilibrium.
__device__ __forceinline__ void lbm_collide(unsigned flags, float &tempC, float &tempN, float &tempS, float &tempE, float &tempW, float &tempT, float &tempB, float &tempNE, float &tempNW, float &tempSE, float &tempSW, float &tempNT, float &tempNB, float &tempST, float &tempSB, float &tempET, float &tempEB, float &tempWT, float &tempWB)
{
    if (flags & LBM_OBSTACLE) {
        float t;
        t = tempN; tempN = tempS; tempS = t;
        t = tempE; tempE = tempW; tempW = t;
        t = tempT; tempT = tempB; tempB = t;
        t = tempNE; tempNE = tempSW; tempSW = t;
        t = tempNW; tempNW = tempSE; tempSE = t;
        t = tempNT; tempNT = tempSB; tempSB = t;
        t = tempNB; tempNB = tempST; tempST = t;
        t = tempET; tempET = tempWB; tempWB = t;
        t = tempEB; tempEB = tempWT; tempWT = t;
    } else {
        float ux, uy, uz, rho, u2, temp1, temp2, temp_base;
        rho = tempC + tempN + tempS + tempE + tempW + tempT + tempB + tempNE + tempNW + tempSE +
              tempSW + tempNT + tempNB + tempST + tempSB + tempET + tempEB + tempWT + tempWB;
        ux = +tempE - tempW + tempNE - tempNW + tempSE - tempSW + tempET + tempEB - tempWT - tempWB;
        uy = +tempN - tempS + tempNE + tempNW - tempSE - tempSW + tempNT + tempNB - tempST - tempSB;
        uz = +tempT - tempB + tempNT - tempNB + tempST - tempSB + tempET - tempEB + tempWT - tempWB;
        ux /= rho;
        uy /= rho;
        uz /= rho;
        if (flags & LBM_ACCEL) {
            ux = 0.005f;
            uy = 0.002f;
            uz = 0.000f;
        }
        u2 = 1.5f * (ux * ux + uy * uy + uz * uz) - 1.0f;
        temp_base = LBM_OMEGA * rho;
        temp1 = LBM_DFL1 * temp_base;
        temp2 = 1.0f - LBM_OMEGA;
        tempC = temp2 * tempC + temp1 * (-u2);
        temp1 = LBM_DFL2 * temp_base;
        tempN = temp2 * tempN + temp1 * (uy * (4.5f * uy + 3.0f) - u2);
        tempS = temp2 * tempS + temp1 * (uy * (4.5f * uy - 3.0f) - u2);
        tempT = temp2 * tempT + temp1 * (uz * (4.5f * uz + 3.0f) - u2);
        tempB = temp2 * tempB + temp1 * (uz * (4.5f * uz - 3.0f) - u2);
        tempE = temp2 * tempE + temp1 * (ux * (4.5f * ux + 3.0f) - u2);
        tempW = temp2 * tempW + temp1 * (ux * (4.5f * ux - 3.0f) - u2);
        temp1 = LBM_DFL3 * temp_base;
        tempNT = temp2 * tempNT + temp1 * ((+uy + uz) * (4.5f * (+uy + uz) + 3.0f) - u2);
        tempNB = temp2 * tempNB + temp1 * ((+uy - uz) * (4.5f * (+uy - uz) + 3.0f) - u2);
        tempST = temp2 * tempST + temp1 * ((-uy + uz) * (4.5f * (-uy + uz) + 3.0f) - u2);
        tempSB = temp2 * tempSB + temp1 * ((-uy - uz) * (4.5f * (-uy - uz) + 3.0f) - u2);
        tempNE = temp2 * tempNE + temp1 * ((+ux + uy) * (4.5f * (+ux + uy) + 3.0f) - u2);
        tempSE = temp2 * tempSE + temp1 * ((+ux - uy) * (4.5f * (+ux - uy) + 3.0f) - u2);
        tempET = temp2 * tempET + temp1 * ((+ux + uz) * (4.5f * (+ux + uz) + 3.0f) - u2);
        tempEB = temp2 * tempEB + temp1 * ((+ux - uz) * (4.5f * (+ux - uz) + 3.0f) - u2);
        tempNW = temp2 * tempNW + temp1 * ((-ux + uy) * (4.5f * (-ux + uy) + 3.0f) - u2);
        tempSW = temp2 * tempSW + temp1 * ((-ux - uy) * (4.5f * (-ux - uy) + 3.0f) - u2);
        tempWT = temp2 * tempWT + temp1 * ((-ux + uz) * (4.5f * (-ux + uz) + 3.0f) - u2);
        tempWB = temp2 * tempWB + temp1 * ((-ux - uz) * (4.5f * (-ux - uz) + 3.0f) - u2);
    }
}

#define TK_LBM_DIRECTIONS(X)                                                                       \
    X(LBM_C, 0, 0, 0, tempC) \
    X(LBM_N, 0, +1, 0, tempN) \
    X(LBM_S, 0, -1, 0, tempS) \
    X(LBM_E, +1, 0, 0, tempE) \
    X(LBM_W, -1, 0, 0, tempW) \
    X(LBM_T, 0, 0, +1, tempT) \
    X(LBM_B, 0, 0, -1, tempB) \
    X(LBM_NE, +1, +1, 0, tempNE) \
    X(LBM_NW, -1, +1, 0, tempNW) \
    X(LBM_SE, +1, -1, 0, tempSE) \
    X(LBM_SW, -1, -1, 0, tempSW) \
    X(LBM_NT, 0, +1, +1, tempNT) \
    X(LBM_NB, 0, +1, -1, tempNB) \
    X(LBM_ST, 0, -1, +1, tempST) \
    X(LBM_SB, 0, -1, -1, tempSB) \
    X(LBM_ET, +1, 0, +1, tempET) \
    X(LBM_EB, +1, 0, -1, tempEB) \
    X(LBM_WT, -1, 0, +1, tempWT) \
    X(LBM_WB, -1, 0, -1, tempWB)

__device__ __forceinline__ void lbm_cell(const float *__restrict__ src, float *__restrict__ dst,
                                         int cells, int c, int sx, int sxy)
{
    float tempC = __builtin_nontemporal_load(src + cells * LBM_C + c);
    float tempN = __builtin_nontemporal_load(src + cells * LBM_N + c);
    float tempS = __builtin_nontemporal_load(src + cells * LBM_S + c);
    float tempE = __builtin_nontemporal_load(src + cells * LBM_E + c);
    float tempW = __builtin_nontemporal_load(src + cells * LBM_W + c);
    float tempT = __builtin_nontemporal_load(src + cells * LBM_T + c);
    float tempB = __builtin_nontemporal_load(src + cells * LBM_B + c);
    float tempNE = __builtin_nontemporal_load(src + cells * LBM_NE + c);
    float tempNW = __builtin_nontemporal_load(src + cells * LBM_NW + c);
    float tempSE = __builtin_nontemporal_load(src + cells * LBM_SE + c);
    float tempSW = __builtin_nontemporal_load(src + cells * LBM_SW + c);
    float tempNT = __builtin_nontemporal_load(src + cells * LBM_NT + c);
    float tempNB = __builtin_nontemporal_load(src + cells * LBM_NB + c);
    float tempST = __builtin_nontemporal_load(src + cells * LBM_ST + c);
    float tempSB = __builtin_nontemporal_load(src + cells * LBM_SB + c);
    float tempET = __builtin_nontemporal_load(src + cells * LBM_ET + c);
    float tempEB = __builtin_nontemporal_load(src + cells * LBM_EB + c);
    float tempWT = __builtin_nontemporal_load(src + cells * LBM_WT + c);
    float tempWB = __builtin_nontemporal_load(src + cells * LBM_WB + c);
    const unsigned flags = __float_as_uint(__builtin_nontemporal_load(src + cells * LBM_FLAGS + c));
    lbm_collide(flags, tempC, tempN, tempS, tempE, tempW, tempT, tempB, tempNE, tempNW, tempSE, tempSW, tempNT, tempNB, tempST, tempSB, tempET, tempEB, tempWT, tempWB);
#define TK_LBM_SCATTER(entry, dx, dy, dz, value)                          \
    do {                                                                  \
        const int t_ = c + (dx) + (dy) * sx + (dz) * sxy;                 \
        if (t_ >= 0 && t_ < cells) dst[cells * (entry) + t_] = (value);   \
    } while (0);
    TK_LBM_DIRECTIONS(TK_LBM_SCATTER)
#undef TK_LBM_SCATTER
}

// Two x-adjacent cells per lane (c even, c + 1 in the same row): every access is 8 bytes
// per lane, which halves the number of vector-memory instructions per byte moved -- the
// per-CU address/data-return unit is what a dword-per-lane streaming kernel saturates first,
// and in a fused launch that unit is shared with the GEMM's loads.  Scatter targets are
// shifted by +-1 cell for 10 of the 19 directions, so the 8-byte accesses are only 4-byte
// aligned; the vector type says so.
typedef float lbm_pair_t __attribute__((ext_vector_type(2), aligned(4)));
// The 20 values of a cell are read once per step and never again: nontemporal loads, so that they pass
// through the L2 without pushing out what has a second use -- the scattered stores, whose lines are
// completed by the waves of neighbouring rows a little later, and in a fused launch the GEMM's operand
// panels.  (Measured at 120 x 120 x 150: the step alone 73.6 instead of 79.5 us in 64-thread workgroups,
// the fused launch with the 4096 x 4096 x 1024 GEMM 95 instead of 113 us.  Nontemporal stores on top
// of that take it back: 96 us alone, 102 us fused.)
__device__ __forceinline__ lbm_pair_t lbm_load_pair(const float *p)
{
    return __builtin_nontemporal_load(reinterpret_cast<const lbm_pair_t *>(p));
}
__device__ __forceinline__ void lbm_store_pair(float *p, lbm_pair_t v)
{
    *reinterpret_cast<lbm_pair_t *>(p) = v;
}

__device__ __forceinline__ void lbm_cell_pair(const float *__restrict__ src, float *__restrict__ dst,
                                              int cells, int c, int sx, int sxy)
{
#define TK_LBM_LOAD(entry, dx, dy, dz, name) \
    const lbm_pair_t name##_in = lbm_load_pair(src + cells * (entry) + c);
    TK_LBM_DIRECTIONS(TK_LBM_LOAD)
#undef TK_LBM_LOAD
    const lbm_pair_t flags_in = lbm_load_pair(src + cells * LBM_FLAGS + c);
#define TK_LBM_SPLIT(entry, dx, dy, dz, name) float name##0 = name##_in.x, name##1 = name##_in.y;
    TK_LBM_DIRECTIONS(TK_LBM_SPLIT)
#undef TK_LBM_SPLIT
    lbm_collide(__float_as_uint(flags_in.x), tempC0, tempN0, tempS0, tempE0, tempW0, tempT0, tempB0, tempNE0, tempNW0, tempSE0, tempSW0, tempNT0, tempNB0, tempST0, tempSB0, tempET0, tempEB0, tempWT0, tempWB0);
    lbm_collide(__float_as_uint(flags_in.y), tempC1, tempN1, tempS1, tempE1, tempW1, tempT1, tempB1, tempNE1, tempNW1, tempSE1, tempSW1, tempNT1, tempNB1, tempST1, tempSB1, tempET1, tempEB1, tempWT1, tempWB1);
#define TK_LBM_SCATTER2(entry, dx, dy, dz, name)                                           \
    do {                                                                                   \
        const int t_ = c + (dx) + (dy) * sx + (dz) * sxy;                                  \
        float *o_ = dst + cells * (entry) + t_;                                            \
        if (t_ >= 0 && t_ + 1 < cells) {                                                   \
            lbm_store_pair(o_, lbm_pair_t{name##0, name##1});            \
        } else {                                                                           \
            if (t_ >= 0 && t_ < cells) o_[0] = name##0;                                    \
            if (t_ + 1 >= 0 && t_ + 1 < cells) o_[1] = name##1;                            \
        }                                                                                  \
    } while (0);
    TK_LBM_DIRECTIONS(TK_LBM_SCATTER2)
#undef TK_LBM_SCATTER2
}

// N rows at once, for a role that has few waves on its CU (inside a fused kernel): all 20 N loads
// of the rows are issued before the first collision, so a wave has N times the bytes in flight.
// Each destination word has one writer whichever rows are taken together, so the result is the
// same as row by row.
template <int N>
__device__ __forceinline__ void lbm_cell_pair_rows(const float *__restrict__ src, float *__restrict__ dst,
                                                   int cells, const int (&c)[N], int sx, int sxy)
{
    lbm_pair_t in[N][20];
#pragma unroll
    for (int r = 0; r < N; ++r) {
#define TK_LBM_LOAD(entry, dx, dy, dz, name) in[r][entry] = lbm_load_pair(src + cells * (entry) + c[r]);
        TK_LBM_DIRECTIONS(TK_LBM_LOAD)
#undef TK_LBM_LOAD
        in[r][LBM_FLAGS] = lbm_load_pair(src + cells * LBM_FLAGS + c[r]);
    }
    // a row is collided and scattered while the loads of the rows behind it are still on their way;
    // the scheduling fences keep the rows' arithmetic apart (interleaved it needs more registers
    // than a fused kernel has)
#pragma unroll
    for (int r = 0; r < N; ++r) {
        __builtin_amdgcn_sched_barrier(0);
#define TK_LBM_SPLIT(entry, dx, dy, dz, name) float name##0 = in[r][entry].x, name##1 = in[r][entry].y;
        TK_LBM_DIRECTIONS(TK_LBM_SPLIT)
#undef TK_LBM_SPLIT
        lbm_collide(__float_as_uint(in[r][LBM_FLAGS].x), tempC0, tempN0, tempS0, tempE0, tempW0, tempT0, tempB0, tempNE0, tempNW0, tempSE0, tempSW0, tempNT0, tempNB0, tempST0, tempSB0, tempET0, tempEB0, tempWT0, tempWB0);
        lbm_collide(__float_as_uint(in[r][LBM_FLAGS].y), tempC1, tempN1, tempS1, tempE1, tempW1, tempT1, tempB1, tempNE1, tempNW1, tempSE1, tempSW1, tempNT1, tempNB1, tempST1, tempSB1, tempET1, tempEB1, tempWT1, tempWB1);
#define TK_LBM_SCATTER_ROW(entry, dx, dy, dz, name)                                        \
    do {                                                                                   \
        const int t_ = c[r] + (dx) + (dy) * sx + (dz) * sxy;                               \
        float *o_ = dst + cells * (entry) + t_;                                            \
        if (t_ >= 0 && t_ + 1 < cells) {                                                   \
            lbm_store_pair(o_, lbm_pair_t{name##0, name##1});                              \
        } else {                                                                           \
            if (t_ >= 0 && t_ < cells) o_[0] = name##0;                                    \
            if (t_ + 1 >= 0 && t_ + 1 < cells) o_[1] = name##1;                            \
        }                                                                                  \
    } while (0);
        TK_LBM_DIRECTIONS(TK_LBM_SCATTER_ROW)
#undef TK_LBM_SCATTER_ROW
    }
    __builtin_amdgcn_sched_barrier(0);
}

// grid_dimension_x = sy, grid_dimension_y = sz, block_dimension_x = sx
// (src/ori_kernel/lbm_kernel.cu:218-222).  ROWS_PER_WAVE = N > 1: a wave takes N of its rows at a
// time (see lbm_cell_pair_rows); which rows a wave owns is the same either way.
template <int ROWS_PER_WAVE = 1>
__device__ __forceinline__ void lbm_role(const float *__restrict__ src, float *__restrict__ dst,
                                         int grid_dimension_x, int grid_dimension_y,
                                         int block_dimension_x, int role_block, int role_blocks,
                                         int start, int end, int tid, int role_threads)
{
    const int sx = block_dimension_x, sy = grid_dimension_x, sz = grid_dimension_y;
    const int sxy = sx * sy;
    const int cells = sxy * sz;
    // even row length: a lane takes two cells, odd: one
    const int per_lane = (sx & 1) ? 1 : 2;
    const int row_lanes = (sx + per_lane - 1) / per_lane;
    const int lanes_per_row = ((row_lanes + TK_WAVE_SIZE - 1) / TK_WAVE_SIZE) * TK_WAVE_SIZE;
    int rows_at_once = role_threads / lanes_per_row;
    int row_slot, x_first, x_step;
    if (rows_at_once >= 1) {
        row_slot = tid / lanes_per_row;
        x_first = (tid % lanes_per_row) * per_lane;
        x_step = lanes_per_row * per_lane;
        if (row_slot >= rows_at_once) return;
    } else {   // row longer than the role: the role's threads sweep it
        rows_at_once = 1;
        row_slot = 0;
        x_first = tid * per_lane;
        x_step = role_threads * per_lane;
    }
    const unsigned stride = (unsigned)role_blocks * rows_at_once;
    unsigned pos = (unsigned)start + role_block * rows_at_once + row_slot;
    if (ROWS_PER_WAVE > 1 && per_lane == 2) {
        constexpr int N = ROWS_PER_WAVE > 1 ? ROWS_PER_WAVE : 2;
        // while N more rows of this wave lie in the range (and the position does not wrap)
        for (; (unsigned long long)pos + (unsigned long long)(N - 1) * stride < (unsigned)end; pos += N * stride) {
            int row[N];
#pragma unroll
            for (int r = 0; r < N; ++r) {
                const unsigned p = pos + (unsigned)r * stride;
                row[r] = (int)(p % sy) * sx + (int)((p / sy) % sz) * sxy;
            }
            for (int x = x_first; x < sx; x += x_step) {
                int c[N];
#pragma unroll
                for (int r = 0; r < N; ++r) c[r] = x + row[r];
                lbm_cell_pair_rows<N>(src, dst, cells, c, sx, sxy);
            }
        }
    }
    for (; pos < (unsigned)end; pos += stride) {
        const int y = pos % sy;
        const int z = (pos / sy) % sz;
        if (per_lane == 2) {
            for (int x = x_first; x < sx; x += x_step)
                lbm_cell_pair(src, dst, cells, x + y * sx + z * sxy, sx, sxy);
        } else {
            for (int x = x_first; x < sx; x += x_step)
                lbm_cell(src, dst, cells, x + y * sx + z * sxy, sx, sxy);
        }
    }
}

}  // namespace tk
