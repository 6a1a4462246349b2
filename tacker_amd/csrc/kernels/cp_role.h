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
//
// 1.0f / sqrtf(r2) is two correctly rounded operations, and the general expansions of an IEEE
// square root and an IEEE divide (scaling for denormals, fix-up of special values) are what the
// kernel's time goes into: about 35 instructions per atom-point pair.  For r2 in
// [2^-20, 2^20) a shorter sequence gives the same two roundings, bit for bit --
//   s0 = v_sqrt(r2); h = 0.5 * v_rcp(s0);            s  = s0 corrected twice by its residual
//   y0 = 2h;                                         y  = y0 after two Newton steps on s
// -- which was checked against sqrtf / divide for every one of the 335 544 320 floats of that
// range (cp_inv_sqrt_selftest below repeats the check on demand).  A wave uses it for an atom
// when all its lanes' r2 are sure to be in the range, and the general expansion otherwise
// (a point within 2^-10 of an atom in y and z, about one atom-row pair in fifty).
#pragma once
#include "role_common.h"
#include "../header/cp_header.h"

__constant__ float4 atominfo[MAXATOMS];

namespace tk {

#define CP_SHORT_LO 9.5367431640625e-07f   // 2^-20
#define CP_SHORT_HI 1048576.0f             // 2^20

// fl(1 / fl(sqrt(r2))) for r2 in [CP_SHORT_LO, CP_SHORT_HI)
__device__ __forceinline__ float cp_inv_sqrt_short(float r2)
{
    const float s0 = __builtin_amdgcn_sqrtf(r2);
    const float h = 0.5f * __builtin_amdgcn_rcpf(s0);
    const float s1 = __builtin_fmaf(__builtin_fmaf(-s0, s0, r2), h, s0);
    const float s = __builtin_fmaf(__builtin_fmaf(-s1, s1, r2), h, s1);
    const float y0 = h + h;
    const float y1 = __builtin_fmaf(__builtin_fmaf(-s, y0, 1.0f), y0, y0);
    return __builtin_fmaf(__builtin_fmaf(-s, y1, 1.0f), y1, y1);
}

template <bool SHORT>
__device__ __forceinline__ float cp_inv_sqrt(float r2)
{
    return SHORT ? cp_inv_sqrt_short(r2) : 1.0f / sqrtf(r2);
}

// true when every lane of the wave may take the short form for this atom: r2 = dx^2 + dyz2 of
// all `points` points of the lane lies in [CP_SHORT_LO, CP_SHORT_HI)
__device__ __forceinline__ bool cp_wave_in_short_range(float dx_first, float dyz2, float reach)
{
    const float far = __builtin_fabsf(dx_first) + reach;
    const bool ok = dyz2 >= CP_SHORT_LO && dyz2 < 0.5f * CP_SHORT_HI && far * far < 0.5f * CP_SHORT_HI;
    return __builtin_amdgcn_ballot_w64(!ok) == 0;
}

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

    const float reach = UNROLLX * gridspacing_u;
    for (int atomid = 0; atomid < numatoms; ++atomid) {
        const float dy = coory - atominfo[atomid].y;
        const float dyz2 = (dy * dy) + atominfo[atomid].z;
        float dx = coorx - atominfo[atomid].x;
        if (cp_wave_in_short_range(dx, dyz2, reach)) {
#pragma unroll
            for (int n = 0; n < UNROLLX; ++n) {
                energyval[n] += atominfo[atomid].w * cp_inv_sqrt<true>(dx * dx + dyz2);
                dx = dx + gridspacing_u;
            }
        } else {
#pragma unroll
            for (int n = 0; n < UNROLLX; ++n) {
                energyval[n] += atominfo[atomid].w * cp_inv_sqrt<false>(dx * dx + dyz2);
                dx = dx + gridspacing_u;
            }
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
    const float reach = UNROLLX * gridspacing_u;
    for (int atomid = 0; atomid < numatoms; ++atomid) {
        const float4 a = atominfo[atomid];
        float dyz2[2], dx[2];
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            const float dy = coory[b] - a.y;
            dyz2[b] = (dy * dy) + a.z;
            dx[b] = coorx[b] - a.x;
        }
        const bool fast = cp_wave_in_short_range(dx[0], dyz2[0], reach) &&
                          cp_wave_in_short_range(dx[1], dyz2[1], reach);
        if (fast) {
#pragma unroll
            for (int b = 0; b < 2; ++b)
#pragma unroll
                for (int n = 0; n < UNROLLX; ++n) {
                    energyval[b][n] += a.w * cp_inv_sqrt<true>(dx[b] * dx[b] + dyz2[b]);
                    dx[b] = dx[b] + gridspacing_u;
                }
        } else {
#pragma unroll
            for (int b = 0; b < 2; ++b)
#pragma unroll
                for (int n = 0; n < UNROLLX; ++n) {
                    energyval[b][n] += a.w * cp_inv_sqrt<false>(dx[b] * dx[b] + dyz2[b]);
                    dx[b] = dx[b] + gridspacing_u;
                }
        }
    }
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int n = 0; n < UNROLLX; ++n) energygrid[outaddr[b] + n * BLOCKSIZEX] += energyval[b][n];
}

// U positions of one x part per thread at once: U blocks, CP_POINTS_PER_POSITION points of
// each.  PART selects the points n in [PART * P, (PART + 1) * P) of the UNROLLX a block's
// thread owns; their dx is reached by the same chain of additions cp_block runs through
// (dx_{n+1} = dx_n + 16 * spacing), so every value equals the one cp_block stores.
template <int U, int PART>
__device__ __forceinline__ void cp_positions(int numatoms, float gridspacing, float *__restrict__ energygrid,
                                             const unsigned (&block)[U], unsigned grid_dimension_x,
                                             unsigned thread_id_x, unsigned thread_id_y)
{
    constexpr int P = CP_POINTS_PER_POSITION;
    unsigned outaddr[U];
    float coory[U], coorx[U];
    float energyval[U][P];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const unsigned xindex = (block[u] % grid_dimension_x) * BLOCKSIZEX * UNROLLX + thread_id_x;
        const unsigned yindex = (block[u] / grid_dimension_x) * BLOCKSIZEY + thread_id_y;
        outaddr[u] = (grid_dimension_x * BLOCKSIZEX * UNROLLX) * yindex + xindex + PART * P * BLOCKSIZEX;
        coory[u] = gridspacing * yindex;
        coorx[u] = gridspacing * xindex;
#pragma unroll
        for (int n = 0; n < P; ++n) energyval[u][n] = 0.0f;
    }
    const float gridspacing_u = gridspacing * BLOCKSIZEX;
    const float reach = P * gridspacing_u;
    for (int atomid = 0; atomid < numatoms; ++atomid) {
        const float4 a = atominfo[atomid];
        float dyz2[U], dx[U];
        bool fast = true;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const float dy = coory[u] - a.y;
            dyz2[u] = (dy * dy) + a.z;
            dx[u] = coorx[u] - a.x;
#pragma unroll
            for (int n = 0; n < PART * P; ++n) dx[u] = dx[u] + gridspacing_u;
            fast = cp_wave_in_short_range(dx[u], dyz2[u], reach) && fast;
        }
        if (fast) {
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int n = 0; n < P; ++n) {
                    energyval[u][n] += a.w * cp_inv_sqrt<true>(dx[u] * dx[u] + dyz2[u]);
                    dx[u] = dx[u] + gridspacing_u;
                }
        } else {
#pragma unroll
            for (int u = 0; u < U; ++u)
#pragma unroll
                for (int n = 0; n < P; ++n) {
                    energyval[u][n] += a.w * cp_inv_sqrt<false>(dx[u] * dx[u] + dyz2[u]);
                    dx[u] = dx[u] + gridspacing_u;
                }
        }
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
        for (int n = 0; n < P; ++n) energygrid[outaddr[u] + n * BLOCKSIZEX] += energyval[u][n];
}

template <int PART>
__device__ __forceinline__ void cp_part_phase(int numatoms, float gridspacing, float *__restrict__ energygrid,
                                              int block_lo, int block_hi, unsigned grid_dimension_x,
                                              int first_owned, int stride, unsigned tx, unsigned ty)
{
    int b = first_owned;
    if (b < block_lo) b += (block_lo - b + stride - 1) / stride * stride;
    // 4, 2 or 1 of the thread's blocks at a time: 8, 4 or 2 independent sqrt/divide chains
    for (; b + 3 * stride < block_hi; b += 4 * stride) {
        const unsigned four[4] = {(unsigned)b, (unsigned)(b + stride), (unsigned)(b + 2 * stride),
                                  (unsigned)(b + 3 * stride)};
        cp_positions<4, PART>(numatoms, gridspacing, energygrid, four, grid_dimension_x, tx, ty);
    }
    if (b + stride < block_hi) {
        const unsigned two[2] = {(unsigned)b, (unsigned)(b + stride)};
        cp_positions<2, PART>(numatoms, gridspacing, energygrid, two, grid_dimension_x, tx, ty);
        b += 2 * stride;
    }
    if (b < block_hi) {
        const unsigned one[1] = {(unsigned)b};
        cp_positions<1, PART>(numatoms, gridspacing, energygrid, one, grid_dimension_x, tx, ty);
    }
}

// Block positions of the GPTB form are a grid of grid_dimension_x * grid_dimension_y
// blocks (the reference's (16,8)-thread blocks of 128 x 8 points) by grid_dimension_z =
// CP_X_PARTS parts: position p does part (p / blocks) % parts of block p % blocks, a part
// being CP_POINTS_PER_POSITION of the UNROLLX points each thread of the block owns -- the
// reference's 3-D index reconstruction (block_id_z = pos / (x * y) % z) over a grid whose z
// splits the unrolled x points, so that a short range of positions is a short piece of
// work.  Every output point is computed whole by one thread, so any split of the grid into
// ranges stores the bits cp_block stores.
//
// A range [start, end) is a partial first row of that grid (one part of some blocks), whole
// rows, and a partial last row.  Every block has one owner thread group for the whole launch
// (slot-major over the role's workgroups), and the owner walks the rows in order: a range
// that runs past the grid and comes round to a point again adds to it a second time, after
// the first.  CP_X_PARTS whole rows that make up all parts of every block are served by the
// whole-block code, two blocks at a time.
__device__ __forceinline__ void cp_role(int numatoms, float gridspacing,
                                        float *__restrict__ energygrid, int grid_dimension_x,
                                        int grid_dimension_y, int grid_dimension_z, int role_block,
                                        int role_blocks, int start, int end, int tid, int role_threads)
{
    constexpr int BLOCK_THREADS = BLOCKSIZEX * BLOCKSIZEY;
    const int blocks_at_once = role_threads / BLOCK_THREADS;
    const int slot = tid / BLOCK_THREADS;
    const int t = tid % BLOCK_THREADS;
    if (slot >= blocks_at_once || start >= end) return;
    const unsigned tx = t % BLOCKSIZEX, ty = t / BLOCKSIZEX;
    const unsigned gx = grid_dimension_x;
    const int blocks = grid_dimension_x * grid_dimension_y;
    const int parts = grid_dimension_z;   // CP_X_PARTS from the host; 1 = whole blocks only
    const int stride = role_blocks * blocks_at_once;
    const int first_owned = slot * role_blocks + role_block;

    const auto part_phase = [&](int lo, int hi, int row) {
        if (parts == 1) {   // a position is a whole block
            int b = first_owned;
            if (b < lo) b += (lo - b + stride - 1) / stride * stride;
            for (; b < hi; b += stride)
                cp_block(numatoms, gridspacing, energygrid, b % gx, b / gx, gx, tx, ty);
            return;
        }
        switch (row % parts) {
        case 0: cp_part_phase<0>(numatoms, gridspacing, energygrid, lo, hi, gx, first_owned, stride, tx, ty); break;
        case 1: cp_part_phase<1>(numatoms, gridspacing, energygrid, lo, hi, gx, first_owned, stride, tx, ty); break;
        case 2: cp_part_phase<2>(numatoms, gridspacing, energygrid, lo, hi, gx, first_owned, stride, tx, ty); break;
        default: cp_part_phase<3>(numatoms, gridspacing, energygrid, lo, hi, gx, first_owned, stride, tx, ty); break;
        }
    };
    const auto whole_blocks = [&]() {   // all parts of every block
        int b = first_owned;
        for (; b + stride < blocks; b += 2 * stride) {
            const unsigned bx[2] = {b % gx, (b + stride) % gx};
            const unsigned by[2] = {b / gx, (b + stride) / gx};
            cp_block_pair(numatoms, gridspacing, energygrid, bx, by, gx, tx, ty);
        }
        if (b < blocks) cp_block(numatoms, gridspacing, energygrid, b % gx, b / gx, gx, tx, ty);
    };

    const int first_row = start / blocks;
    const int last_row = (end - 1) / blocks;
    if (first_row == last_row) {
        part_phase(start - first_row * blocks, end - first_row * blocks, first_row);
        return;
    }
    int row = first_row;
    if (start != first_row * blocks) {
        part_phase(start - first_row * blocks, blocks, row);
        ++row;
    }
    const int whole_end = (end == (last_row + 1) * blocks) ? last_row + 1 : last_row;
    while (row < whole_end) {
        if (parts > 1 && row % parts == 0 && row + parts <= whole_end) {
            whole_blocks();
            row += parts;
        } else {
            part_phase(0, blocks, row);
            ++row;
        }
    }
    if (whole_end == last_row) part_phase(0, end - last_row * blocks, last_row);
}

}  // namespace tk
