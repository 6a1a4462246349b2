// Nearest-neighbour role (Rodinia nn): the Euclidean distance of every record's (lat, lng) to one
// query point.
//
// Replaces ori_nn / general_ptb_nn (src/ori_kernel/nn_kernel.cu:9-17,
// src/gptb_kernel/nn_kernel.cu:3-23 of the reference).  A block position is one block of the
// reference's launch: block_dimension_x consecutive records starting at
//   block_dimension_x * (grid_dimension_x * block_id_y + block_id_x)
// (the ori kernel's globalId; the reference's GPTB form multiplies block_id_x by block_id_y
// instead, which is not what its own unfused kernel computes -- this role follows the unfused one),
// records past numRecords left alone.  Per record, in fp32 and in this order:
//   dlat = lat - r.lat;  dlng = lng - r.lng;  dist = sqrtf(dlat * dlat + dlng * dlng)
// with an IEEE square root, so the output is bit-identical to a CPU evaluation.
//
// gfx950: a pure stream, 8 bytes in and 4 out per record.  A lane takes one record of a position
// (a wave reads 512 contiguous bytes and writes 256) and the role's threads serve
// role_threads / block_dimension_x positions at a time, four such steps in flight before the
// first store so that a wave keeps 2 KiB of loads outstanding.
#pragma once
#include "role_common.h"
#include "../header/nn_header.h"

namespace tk {

__device__ __forceinline__ float nn_distance(float2 r, float lat, float lng)
{
    const float dlat = lat - r.x;
    const float dlng = lng - r.y;
    return sqrtf(dlat * dlat + dlng * dlng);
}

// Block positions [start, end) of the grid (grid_dimension_x, grid_dimension_y) are served by the
// role's role_blocks persistent workgroups in turn; a position past the grid wraps as the
// reference's block_pos % grid_dimension_x, (block_pos / grid_dimension_x) % grid_dimension_y do.
__device__ __forceinline__ void nn_role(const LatLong *__restrict__ d_locations, float *__restrict__ d_distances,
                                        int numRecords, float lat, float lng, int grid_dimension_x,
                                        int grid_dimension_y, int block_dimension_x, int role_block, int role_blocks,
                                        int start, int end, int tid, int role_threads)
{
    constexpr int DEPTH = 4;
    if (start >= end || grid_dimension_x <= 0 || grid_dimension_y <= 0 || block_dimension_x <= 0) return;
    const float2 *__restrict__ records = reinterpret_cast<const float2 *>(d_locations);
    // positions served at once and this thread's place among them
    const int width = block_dimension_x;
    const int at_once = role_threads >= width ? role_threads / width : 1;
    const int group = role_threads >= width ? tid / width : 0;
    const int first = role_threads >= width ? tid % width : tid;
    const int step = role_threads >= width ? width : role_threads;
    if (group >= at_once) return;
    for (int j = group;; j += DEPTH * at_once) {
        long long base[DEPTH];
        bool live[DEPTH];
#pragma unroll
        for (int u = 0; u < DEPTH; ++u) {
            const long long pos = (long long)start + role_block + (long long)(j + u * at_once) * role_blocks;
            live[u] = pos < end;
            const unsigned p = (unsigned)pos;
            const unsigned bx = p % (unsigned)grid_dimension_x;
            const unsigned by = (p / (unsigned)grid_dimension_x) % (unsigned)grid_dimension_y;
            base[u] = (long long)width * ((long long)grid_dimension_x * by + bx);
        }
        if (!live[0]) return;
        for (int r = first; r < width; r += step) {
            float2 v[DEPTH];
#pragma unroll
            for (int u = 0; u < DEPTH; ++u)
                if (live[u] && base[u] + r < numRecords) v[u] = records[base[u] + r];
#pragma unroll
            for (int u = 0; u < DEPTH; ++u)
                if (live[u] && base[u] + r < numRecords) d_distances[base[u] + r] = nn_distance(v[u], lat, lng);
        }
        if (!live[DEPTH - 1]) return;
    }
}

}  // namespace tk
