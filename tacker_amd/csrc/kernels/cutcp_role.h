// Cutoff Coulomb potential role: the potential of binned point charges on a lattice, every charge
// acting within the cutoff only (src/ori_kernel/cutcp_kernel.cu:19-158,
// src/gptb_kernel/cutcp_kernel.cu:12-183 of the reference).
//
// A block position is a region of 8 x 8 x 8 lattice points.  The reference gives it to a block of
// 128 threads (8, 2, 8): thread (tx, ty, tz) owns the points (tx, ty + 2 e, tz), e = 0 .. 3, and all
// threads walk the same atoms -- the bins the neighbour list names around the region's centre bin,
// staged 32 bins at a time in shared memory between two block barriers.  Here the atoms of a bin are
// the same for every lane of a wavefront, so they arrive by scalar loads (one bin = 128 bytes) and
// there is nothing to stage or to wait for: a wavefront plays 64 of the 128 threads and serves
// half a region on its own, which is what lets the role live in a fused kernel next to roles that
// own the workgroup barrier.  Per lane the arithmetic and its order are the reference's:
//   dx = ax - x; dz = az - z; dxdz2 = dx*dx + dz*dz; dy = ay - y; r2 = dy*dy + dxdz2;
//   if (r2 < cutoff2) { s = 1 - r2 * inv_cutoff2; energy += aq * rsqrt(r2) * s * s; }  dy -= 2h; ...
// with the hardware's reciprocal square root where the reference has CUDA's rsqrtf (both are
// approximations of about one unit in the last place: results agree within rounding, not bit for bit).
#pragma once
#include "role_common.h"
#include "../header/cutcp_header.h"

// the neighbour list: offsets (i, j, k) of the bins to visit around a region's centre bin
// (cudaMemcpyToSymbol(NbrListLen / NbrList, ...), src/ori_kernel/cutcp_kernel.cu:12-13,241-242)
__constant__ int NbrListLen;
__constant__ int NbrList[NBRLIST_MAXLEN][3];

namespace tk {

typedef __attribute__((address_space(4))) const float4_t cutcp_const_float4;

// half `half` of region (xr, yr, zr): the reference's threads 64 half + lane
__device__ __forceinline__ void cutcp_half_region(int binDim_x, int binDim_y, const float *binZeroAddr, float h,
                                                  float cutoff2, float inv_cutoff2, float *regionZeroAddr, int gdx,
                                                  int gdy, int xr, int yr, int zr, int half, int lane)
{
    const int tid = 64 * half + lane;
    const int tx = tid & 7, ty = (tid >> 3) & 1, tz = tid >> 4;
    float *region = regionZeroAddr + (size_t)((zr * gdy + yr) * gdx + xr) * REGION_SIZE;
    const float x = (8 * xr + tx) * h;
    const float y = (8 * yr + ty) * h;
    const float z = (8 * zr + tz) * h;
    // bin of the region's centre
    const int bx = (int)floorf((8 * xr + 4) * h * BIN_INVLEN);
    const int by = (int)floorf((8 * yr + 4) * h * BIN_INVLEN);
    const int bz = (int)floorf((8 * zr + 4) * h * BIN_INVLEN);
    const float two_h = 2.0f * h;
    float energy0 = 0.f, energy1 = 0.f, energy2 = 0.f, energy3 = 0.f;
    const int len = NbrListLen;
    for (int n = 0; n < len; ++n) {
        const int i = bx + NbrList[n][0];
        const int j = by + NbrList[n][1];
        const int k = bz + NbrList[n][2];
        const long long bin = ((long long)(k * binDim_y + j) * binDim_x + i) * BIN_DEPTH;
        // wave-uniform address of read-only data: scalar loads
        const cutcp_const_float4 *atoms =
            (const cutcp_const_float4 *)(reinterpret_cast<const float4_t *>(binZeroAddr) + bin);
#pragma unroll
        for (int a = 0; a < BIN_DEPTH; ++a) {
            const float4_t atom = atoms[a];
            const float aq = atom.w;
            if (0.f == aq) break;   // no more atoms in this bin
            const float dx = atom.x - x;
            const float dz = atom.z - z;
            const float dxdz2 = dx * dx + dz * dz;
            float dy = atom.y - y;
            float r2 = dy * dy + dxdz2;
            if (r2 < cutoff2) {
                const float s = (1.f - r2 * inv_cutoff2);
                energy0 += aq * __builtin_amdgcn_rsqf(r2) * s * s;
            }
            dy -= two_h;
            r2 = dy * dy + dxdz2;
            if (r2 < cutoff2) {
                const float s = (1.f - r2 * inv_cutoff2);
                energy1 += aq * __builtin_amdgcn_rsqf(r2) * s * s;
            }
            dy -= two_h;
            r2 = dy * dy + dxdz2;
            if (r2 < cutoff2) {
                const float s = (1.f - r2 * inv_cutoff2);
                energy2 += aq * __builtin_amdgcn_rsqf(r2) * s * s;
            }
            dy -= two_h;
            r2 = dy * dy + dxdz2;
            if (r2 < cutoff2) {
                const float s = (1.f - r2 * inv_cutoff2);
                energy3 += aq * __builtin_amdgcn_rsqf(r2) * s * s;
            }
        }
    }
    float *mine = region + (tid >> 4) * 64 + (tid & 15);
    mine[0] = energy0;
    mine[16] = energy1;
    mine[32] = energy2;
    mine[48] = energy3;
}

// grid_dimension_x/y/z: regions along x, y, z.  Position p is region (p / (gdy gdz), (p / gdz) % gdy,
// p % gdz) (src/gptb_kernel/cutcp_kernel.cu:61-63); the half regions of [start, end) go to the role's
// wavefronts in turn.
__device__ __forceinline__ void cutcp_role(int binDim_x, int binDim_y, const float *binZeroAddr, float h, float cutoff2,
                                           float inv_cutoff2, float *regionZeroAddr, int grid_dimension_x,
                                           int grid_dimension_y, int grid_dimension_z, int role_block, int role_blocks,
                                           int start, int end, int tid, int role_threads)
{
    const int waves = role_threads / 64;
    const int wave = tid / 64;
    if (wave >= waves || start >= end) return;
    const int lane = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    const int items = 2 * (end - start);
    const int stride = role_blocks * waves;
    for (int it = role_block + role_blocks * wave; it < items; it += stride) {
        const int itu = __builtin_amdgcn_readfirstlane(it);
        const int pos = start + (itu >> 1);
        const int yz = grid_dimension_y * grid_dimension_z;
        const int xr = (pos / yz) % grid_dimension_x;
        const int yr = (pos / grid_dimension_z) % grid_dimension_y;
        const int zr = pos % grid_dimension_z;
        cutcp_half_region(binDim_x, binDim_y, binZeroAddr, h, cutoff2, inv_cutoff2, regionZeroAddr, grid_dimension_x,
                          grid_dimension_y, xr, yr, zr, itu & 1, lane);
    }
}

}  // namespace tk
