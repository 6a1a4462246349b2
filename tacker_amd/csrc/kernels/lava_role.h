// lavaMD role (Rodinia): for every particle of a home box, the potential and force it feels from
// the particles of the home box and of its up to 26 neighbour boxes,
//   r2 = vi + vj - (xi xj + yi yj + zi zj);  vij = exp(-a2 r2);  fs = 2 vij;
//   f.v += qj vij;  f.x += qj fs (xi - xj);  f.y, f.z likewise,        a2 = 2 alpha^2,
// accumulated onto the force array in the order home box, neighbour 1, 2, ... and particle 0 .. 99
// within a box.
//
// Replaces ori_lava / general_ptb_lava (src/ori_kernel/lava_kernel.cu:9-141,
// src/gptb_kernel/lava_kernel.cu:3-140 of the reference).  The reference gives a home box to a
// block of 128 threads and stages the home and the neighbour particles in shared memory between
// block barriers.  All threads walk the same neighbour particles, so here they are wave-uniform
// data and arrive by scalar loads (through a constant-address-space pointer, as the atoms of cp
// and cutcp do): no LDS, no barrier, and a wavefront serves a box on its own, a lane holding
// particles lane and lane + 64 of the 100.  fp32 in the source's order, each operation rounded by
// itself; the exponential is the hardware's 2^x of -u2 log2(e) where the reference calls CUDA's
// expf: results agree within a tolerance, not bit for bit.
//
// Block positions.  A box through its 27 boxes is 270 000 pair interactions, 180 us of one
// wavefront and far longer than a GEMM, so -- as for cutcp -- the position grid has a second
// dimension: position p adds part (p / boxes) % 27 (0 = the home box, k = neighbour k of the
// box's list; nothing where the box has fewer neighbours) to box p % boxes.  The forces rest in the
// output between parts.  Every box has one owner wavefront for the whole launch, which walks the
// rows of the grid in order, so a box's parts are added in ascending order without any
// synchronisation and whole rows that follow each other are one run through their parts.
#pragma once
#include "role_common.h"
#include "../header/lava_header.h"

namespace tk {

typedef __attribute__((address_space(4))) const float4_t lava_const_float4;
typedef __attribute__((address_space(4))) const float lava_const_float;
typedef __attribute__((address_space(4))) const box_str lava_const_box;

struct LavaParticle {
    float4_t r;   // v, x, y, z
    float4_t f;   // running potential and force
};

// the contribution of neighbour particle (rb, qb) to one home particle
__device__ __forceinline__ void lava_pair(LavaParticle &a, const float4_t rb, const float qb, const float a2)
{
    const float r2 = a.r[0] + rb[0] - (a.r[1] * rb[1] + a.r[2] * rb[2] + a.r[3] * rb[3]);
    const float u2 = a2 * r2;
    const float vij = __builtin_amdgcn_exp2f(-u2 * 1.44269504088896340736f);
    const float fs = 2.0f * vij;
    const float fxij = fs * (a.r[1] - rb[1]);
    const float fyij = fs * (a.r[2] - rb[2]);
    const float fzij = fs * (a.r[3] - rb[3]);
    a.f[0] += qb * vij;
    a.f[1] += qb * fxij;
    a.f[2] += qb * fyij;
    a.f[3] += qb * fzij;
}

// box `bx`, parts [part_begin, part_end) of its list, by one wavefront
__device__ __forceinline__ void lava_box(const float a2, const box_str *d_box_gpu, const FOUR_VECTOR *d_rv_gpu,
                                         const float *d_qv_gpu, FOUR_VECTOR *d_fv_gpu, int bx, int part_begin,
                                         int part_end, int lane)
{
    const lava_const_box *boxes = (const lava_const_box *)d_box_gpu;
    const long first_i = boxes[bx].offset;
    const int neighbours = boxes[bx].nn;
    if (part_end > 1 + neighbours) part_end = 1 + neighbours;
    if (part_begin >= part_end) return;
    const bool second = lane + 64 < NUMBER_PAR_PER_BOX;   // lanes 0 .. 35 hold two particles
    const float4_t *rA = reinterpret_cast<const float4_t *>(d_rv_gpu + first_i);
    float4_t *fA = reinterpret_cast<float4_t *>(d_fv_gpu + first_i);
    LavaParticle p0, p1;
    p0.r = rA[lane];
    p0.f = fA[lane];
    p1.r = second ? rA[lane + 64] : float4_t{0.f, 0.f, 0.f, 0.f};
    p1.f = second ? fA[lane + 64] : float4_t{0.f, 0.f, 0.f, 0.f};
    for (int k = part_begin; k < part_end; ++k) {
        const int pointer = k == 0 ? bx : boxes[bx].nei[k - 1].number;
        const long first_j = boxes[pointer].offset;
        const lava_const_float4 *rB = (const lava_const_float4 *)(d_rv_gpu + first_j);
        const lava_const_float *qB = (const lava_const_float *)(d_qv_gpu + first_j);
#pragma unroll 4
        for (int j = 0; j < NUMBER_PAR_PER_BOX; ++j) {
            const float4_t rb = rB[j];
            const float qb = qB[j];
            lava_pair(p0, rb, qb, a2);
            lava_pair(p1, rb, qb, a2);
        }
    }
    fA[lane] = p0.f;
    if (second) fA[lane + 64] = p1.f;
}

// One phase of a launch: boxes [box_lo, box_hi) each walk parts [part_begin, part_end).  A
// wavefront serves the boxes it owns: first_owned, first_owned + stride, ...
__device__ __forceinline__ void lava_phase(int box_lo, int box_hi, int part_begin, int part_end, const float a2,
                                           const box_str *d_box_gpu, const FOUR_VECTOR *d_rv_gpu,
                                           const float *d_qv_gpu, FOUR_VECTOR *d_fv_gpu, int first_owned, int stride,
                                           int lane)
{
    if (box_lo >= box_hi || part_begin >= part_end) return;
    int c = first_owned;
    if (c < box_lo) c += (box_lo - c + stride - 1) / stride * stride;
    for (; c < box_hi; c += stride)
        lava_box(a2, d_box_gpu, d_rv_gpu, d_qv_gpu, d_fv_gpu, __builtin_amdgcn_readfirstlane(c), part_begin, part_end,
                 lane);
}

// grid_dimension_x: boxes (the reference's grid); the position grid has the boxes as columns and the
// LAVA_PARTS parts as rows.  A range that runs past the grid wraps.
__device__ __forceinline__ void lava_role(par_str d_par_gpu, dim_str d_dim_gpu, const box_str *d_box_gpu,
                                          const FOUR_VECTOR *d_rv_gpu, const float *d_qv_gpu, FOUR_VECTOR *d_fv_gpu,
                                          int grid_dimension_x, int role_block, int role_blocks, int start, int end,
                                          int tid, int role_threads)
{
    const int waves = role_threads / TK_WAVE_SIZE;
    const int wave = tid / TK_WAVE_SIZE;
    if (wave >= waves || start >= end) return;
    const int lane = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    // boxes past number_boxes do nothing in the reference (src/ori_kernel/lava_kernel.cu:21)
    const int gx = (long)grid_dimension_x < d_dim_gpu.number_boxes ? grid_dimension_x : (int)d_dim_gpu.number_boxes;
    if (gx <= 0 || grid_dimension_x <= 0) return;
    const float a2 = 2.0 * d_par_gpu.alpha * d_par_gpu.alpha;
    const int gy = LAVA_PARTS;
    const int cols = grid_dimension_x;   // positions per row, including boxes past number_boxes
    const int stride = role_blocks * waves;
    const int first_owned = wave * role_blocks + role_block;
#define LAVA_PHASE(lo_, hi_, pb_, pe_)                                                                       \
    lava_phase(lo_, min(hi_, gx), pb_, pe_, a2, d_box_gpu, d_rv_gpu, d_qv_gpu, d_fv_gpu, first_owned, stride, lane)
    const int first_row = start / cols;
    const int last_row = (end - 1) / cols;
    if (first_row == last_row) {
        LAVA_PHASE(start - first_row * cols, end - first_row * cols, first_row % gy, first_row % gy + 1);
        return;
    }
    int row = first_row;
    if (start != first_row * cols) {   // partial first row
        LAVA_PHASE(start - first_row * cols, cols, row % gy, row % gy + 1);
        ++row;
    }
    const int whole_end = (end == (last_row + 1) * cols) ? last_row + 1 : last_row;   // whole rows [row, whole_end)
    while (row < whole_end) {
        // rows up to the next multiple of the part count are consecutive parts: one run
        const int run_end = min(whole_end, (row / gy + 1) * gy);
        LAVA_PHASE(0, cols, row % gy, (run_end - 1) % gy + 1);
        row = run_end;
    }
    if (whole_end == last_row)   // partial last row
        LAVA_PHASE(0, end - last_row * cols, last_row % gy, last_row % gy + 1);
#undef LAVA_PHASE
}

}  // namespace tk
