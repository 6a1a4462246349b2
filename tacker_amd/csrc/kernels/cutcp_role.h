// Cutoff Coulomb potential role: the potential of binned point charges on a lattice, every charge
// acting within the cutoff only (src/ori_kernel/cutcp_kernel.cu:19-158,
// src/gptb_kernel/cutcp_kernel.cu:12-183 of the reference).
//
// The reference's block position is a region of 8 x 8 x 8 lattice points, given to a block of
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

// half `half` of region (xr, yr, zr): the reference's threads 64 half + lane, over parts
// [part_begin, part_end) of the neighbour list of `len` entries; part p of `parts` holds the entries
// p, p + parts, p + 2 parts, ... (every part a sample of the whole neighbourhood, so that parts cost
// the same wherever the atoms are).  A range that does not start with part 0 goes on from the
// energies in memory, where the range before it left them (a float stored and reloaded is unchanged,
// so consecutive ranges give the bits of one walk through all parts).
//
// AHEAD = false: the atoms of a bin by scalar loads, issued when the bin's turn comes -- the faster
// form when the SIMD has other waves to run meanwhile (the plain kernel: 300 against 330 us).
// AHEAD = true: the 32 floats of a bin in 32 lanes of one register, fetched with one vector load
// while the bin before it is walked, the atoms handed out with v_readlane -- a wave that has its
// SIMD almost to itself (a slice of positions next to a GEMM) does not wait for the L2 once per
// bin.  The atoms' bits, and so the results, are the same either way.
template <bool AHEAD>
__device__ __forceinline__ void cutcp_half_region(int binDim_x, int binDim_y, const float *binZeroAddr, float h,
                                                  float cutoff2, float inv_cutoff2, float *regionZeroAddr, int gdx,
                                                  int gdy, int xr, int yr, int zr, int half, int lane, int part_begin,
                                                  int part_end, int parts, int len)
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
    float *mine = region + (tid >> 4) * 64 + (tid & 15);
    float energy0 = 0.f, energy1 = 0.f, energy2 = 0.f, energy3 = 0.f;
    if (part_begin > 0) {
        energy0 = mine[0];
        energy1 = mine[16];
        energy2 = mine[32];
        energy3 = mine[48];
    }
    const float4_t *bins = reinterpret_cast<const float4_t *>(binZeroAddr);
    const auto bin_of = [&](int n) -> const float4_t * {
        const int i = bx + NbrList[n][0];
        const int j = by + NbrList[n][1];
        const int k = bz + NbrList[n][2];
        return bins + ((long long)(k * binDim_y + j) * binDim_x + i) * BIN_DEPTH;
    };
    const auto lane_of = [](float v, int l) -> float {
        return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), l));
    };
// one atom {ax_, ay_, az_, aq_} (wave-uniform) against the lane's four points
#define CUTCP_ATOM(ax_, ay_, az_, aq_)                                                            \
    {                                                                                             \
        const float dx = (ax_) - x;                                                               \
        const float dz = (az_) - z;                                                               \
        const float dxdz2 = dx * dx + dz * dz;                                                    \
        float dy = (ay_) - y;                                                                     \
        float r2 = dy * dy + dxdz2;                                                               \
        if (r2 < cutoff2) {                                                                       \
            const float s = (1.f - r2 * inv_cutoff2);                                             \
            energy0 += (aq_) * __builtin_amdgcn_rsqf(r2) * s * s;                                 \
        }                                                                                         \
        dy -= two_h;                                                                              \
        r2 = dy * dy + dxdz2;                                                                     \
        if (r2 < cutoff2) {                                                                       \
            const float s = (1.f - r2 * inv_cutoff2);                                             \
            energy1 += (aq_) * __builtin_amdgcn_rsqf(r2) * s * s;                                 \
        }                                                                                         \
        dy -= two_h;                                                                              \
        r2 = dy * dy + dxdz2;                                                                     \
        if (r2 < cutoff2) {                                                                       \
            const float s = (1.f - r2 * inv_cutoff2);                                             \
            energy2 += (aq_) * __builtin_amdgcn_rsqf(r2) * s * s;                                 \
        }                                                                                         \
        dy -= two_h;                                                                              \
        r2 = dy * dy + dxdz2;                                                                     \
        if (r2 < cutoff2) {                                                                       \
            const float s = (1.f - r2 * inv_cutoff2);                                             \
            energy3 += (aq_) * __builtin_amdgcn_rsqf(r2) * s * s;                                 \
        }                                                                                         \
    }
    if (AHEAD) {
        // entry of the walk after (part, n): n + parts, or the first entry of the next part
        int part = part_begin, n = part_begin;
        while (part < part_end && n >= len) n = ++part;   // parts beyond a short list are empty
        float cur = part < part_end ? reinterpret_cast<const float *>(bin_of(n))[lane & 31] : 0.f;
        while (part < part_end) {
            int part_next = part, n_next = n + parts;
            while (part_next < part_end && n_next >= len) n_next = ++part_next;
            const float nxt = part_next < part_end ? reinterpret_cast<const float *>(bin_of(n_next))[lane & 31] : 0.f;
#pragma unroll
            for (int a = 0; a < BIN_DEPTH; ++a) {
                const float aq = lane_of(cur, 4 * a + 3);
                if (0.f == aq) break;   // no more atoms in this bin
                CUTCP_ATOM(lane_of(cur, 4 * a), lane_of(cur, 4 * a + 1), lane_of(cur, 4 * a + 2), aq)
            }
            cur = nxt;
            part = part_next;
            n = n_next;
        }
    } else {
        for (int part = part_begin; part < part_end; ++part) {
            for (int n = part; n < len; n += parts) {
                // wave-uniform address of read-only data: scalar loads
                const cutcp_const_float4 *atoms = (const cutcp_const_float4 *)bin_of(n);
#pragma unroll
                for (int a = 0; a < BIN_DEPTH; ++a) {
                    const float4_t atom = atoms[a];
                    const float aq = atom.w;
                    if (0.f == aq) break;   // no more atoms in this bin
                    CUTCP_ATOM(atom.x, atom.y, atom.z, aq)
                }
            }
        }
    }
#undef CUTCP_ATOM
    mine[0] = energy0;
    mine[16] = energy1;
    mine[32] = energy2;
    mine[48] = energy3;
}

// One phase of a launch: regions [region_lo, region_hi) (in position order) each walk parts
// [part_begin, part_end) of the neighbour list.  A wavefront serves the half regions it owns: first_owned,
// first_owned + stride, ...
template <bool AHEAD>
__device__ __forceinline__ void cutcp_phase(int region_lo, int region_hi, int part_begin, int part_end, int parts,
                                            int len, int binDim_x,
                                            int binDim_y, const float *binZeroAddr, float h, float cutoff2,
                                            float inv_cutoff2, float *regionZeroAddr, int gdx, int gdy, int gdz,
                                            int first_owned, int stride, int lane)
{
    if (region_lo >= region_hi || part_begin >= part_end) return;
    const int lo = 2 * region_lo, hi = 2 * region_hi;
    int c = first_owned;
    if (c < lo) c += (lo - c + stride - 1) / stride * stride;
    for (; c < hi; c += stride) {
        const int cu = __builtin_amdgcn_readfirstlane(c);
        const int r = cu >> 1;
        // region r of the reference's GPTB order, x slowest (src/gptb_kernel/cutcp_kernel.cu:61-63)
        cutcp_half_region<AHEAD>(binDim_x, binDim_y, binZeroAddr, h, cutoff2, inv_cutoff2, regionZeroAddr, gdx, gdy,
                                 r / (gdy * gdz), (r / gdz) % gdy, r % gdz, cu & 1, lane, part_begin, part_end, parts, len);
    }
}

// grid_dimension_x, _y: regions along x and y; grid_dimension_z: regions along z times the parts of
// the neighbour list (ceil(NbrListLen / CUTCP_NBR_CHUNK) parts of at most CUTCP_NBR_CHUNK entries, dealt
// round-robin; 1 part when the list is empty).  The position grid has the regions as columns and the
// parts as rows: position p adds part (p / regions) % parts to region p % regions.  Every half region has one owner wavefront for the
// whole launch, which walks the rows in order, so the parts of a region are added in ascending order
// without any synchronisation, whole rows that follow each other are one run through their parts, and
// a range that runs past the grid wraps.
template <bool AHEAD = false>
__device__ __forceinline__ void cutcp_role(int binDim_x, int binDim_y, const float *binZeroAddr, float h, float cutoff2,
                                           float inv_cutoff2, float *regionZeroAddr, int grid_dimension_x,
                                           int grid_dimension_y, int grid_dimension_z, int role_block, int role_blocks,
                                           int start, int end, int tid, int role_threads)
{
    const int waves = role_threads / 64;
    const int wave = tid / 64;
    if (wave >= waves || start >= end) return;
    const int lane = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    const int len = NbrListLen;
    const int gy = max(1, (len + CUTCP_NBR_CHUNK - 1) / CUTCP_NBR_CHUNK);   // parts = rows
    const int gdz = grid_dimension_z / gy;                                     // regions along z
    const int gx = grid_dimension_x * grid_dimension_y * gdz;                  // regions = columns
    if (gx <= 0) return;
    const int stride = role_blocks * waves;
    const int first_owned = wave * role_blocks + role_block;
    const auto chunk_begin = [&](int row) { return row % gy; };
    const auto chunk_end = [&](int row) { return row % gy + 1; };
#define CUTCP_PHASE(lo_, hi_, pb_, pe_)                                                                          \
    cutcp_phase<AHEAD>(lo_, hi_, pb_, pe_, gy, len, binDim_x, binDim_y, binZeroAddr, h, cutoff2, inv_cutoff2,           \
                regionZeroAddr, grid_dimension_x, grid_dimension_y, gdz, first_owned, stride, lane)
    const int first_row = start / gx;
    const int last_row = (end - 1) / gx;
    if (first_row == last_row) {
        CUTCP_PHASE(start - first_row * gx, end - first_row * gx, chunk_begin(first_row), chunk_end(first_row));
        return;
    }
    int row = first_row;
    if (start != first_row * gx) {   // partial first row
        CUTCP_PHASE(start - first_row * gx, gx, chunk_begin(row), chunk_end(row));
        ++row;
    }
    const int whole_end = (end == (last_row + 1) * gx) ? last_row + 1 : last_row;   // whole rows [row, whole_end)
    while (row < whole_end) {
        // rows up to the next multiple of the part count are consecutive parts: one run
        const int run_end = min(whole_end, (row / gy + 1) * gy);
        CUTCP_PHASE(0, gx, chunk_begin(row), chunk_end(run_end - 1));
        row = run_end;
    }
    if (whole_end == last_row)       // partial last row
        CUTCP_PHASE(0, end - last_row * gx, chunk_begin(last_row), chunk_end(last_row));
#undef CUTCP_PHASE
}

}  // namespace tk
