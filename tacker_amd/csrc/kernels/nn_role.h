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
// gfx950: a pure stream, 8 bytes in and 4 out per record.  A lane takes two adjacent records of a
// position (16 bytes in, 8 out; one record where the block width is odd or the arrays are not
// 16-byte aligned), the role's threads serve as many positions at a time as they have lanes for,
// and four such steps are in flight before the first store so that a wave keeps 4 KiB of loads
// outstanding.
#pragma once
#include "role_common.h"
#include "../header/nn_header.h"

// steps of loads a lane issues before its first store
#ifndef NN_STEPS_IN_FLIGHT
#define NN_STEPS_IN_FLIGHT 4
#endif

namespace tk {

__device__ __forceinline__ float nn_distance(float2 r, float lat, float lng)
{
    const float dlat = lat - r.x;
    const float dlng = lng - r.y;
    return sqrtf(dlat * dlat + dlng * dlng);
}

// PER records per lane (1 or 2)
template <int PER>
__device__ __forceinline__ void nn_positions(const float *__restrict__ records, float *__restrict__ d_distances,
                                             int numRecords, float lat, float lng, int grid_dimension_x,
                                             int grid_dimension_y, int width, int role_block, int role_blocks,
                                             int start, int end, int tid, int role_threads)
{
    constexpr int DEPTH = NN_STEPS_IN_FLIGHT;
    typedef float vec_in __attribute__((ext_vector_type(2 * PER)));
    // lanes a position takes, positions served at once and this thread's place among them
    const int lanes = (width + PER - 1) / PER;
    const int at_once = role_threads >= lanes ? role_threads / lanes : 1;
    const int group = role_threads >= lanes ? tid / lanes : 0;
    const int first = role_threads >= lanes ? tid % lanes : tid;
    const int step = role_threads >= lanes ? lanes : role_threads;
    if (group >= at_once) return;
    for (int j = group;; j += DEPTH * at_once) {
        long long base[DEPTH];
        bool live[DEPTH];
#pragma unroll
        for (int u = 0; u < DEPTH; ++u) {
            const long long pos = (long long)start + role_block + (long long)(j + u * at_once) * role_blocks;
            live[u] = pos < end;
            const unsigned q = (unsigned)pos;
            const unsigned bx = q % (unsigned)grid_dimension_x;
            const unsigned by = (q / (unsigned)grid_dimension_x) % (unsigned)grid_dimension_y;
            base[u] = (long long)width * ((long long)grid_dimension_x * by + bx);
        }
        if (!live[0]) return;
        for (int l = first; l < lanes; l += step) {
            const int r = PER * l;
            vec_in v[DEPTH];
            bool whole[DEPTH];   // all PER records of the lane exist
#pragma unroll
            for (int u = 0; u < DEPTH; ++u) {
                whole[u] = live[u] && base[u] + r + PER <= numRecords;
                // records are read once and distances written once, 7.9 GB that nothing reads again soon:
                // nontemporal both ways (1.54 instead of 1.61 ms at 655 360 000 records; only the loads:
                // 1.74-1.78 ms, only the stores: no change)
                if (whole[u]) v[u] = __builtin_nontemporal_load(reinterpret_cast<const vec_in *>(records + 2 * (base[u] + r)));
            }
#pragma unroll
            for (int u = 0; u < DEPTH; ++u) {
                if (whole[u]) {
                    if constexpr (PER == 2) {
                        float2 d;
                        d.x = nn_distance(float2{v[u][0], v[u][1]}, lat, lng);
                        d.y = nn_distance(float2{v[u][2], v[u][3]}, lat, lng);
                        typedef float nn_f2 __attribute__((ext_vector_type(2)));
                        __builtin_nontemporal_store(nn_f2{d.x, d.y}, reinterpret_cast<nn_f2 *>(d_distances + base[u] + r));
                    } else {
                        d_distances[base[u] + r] = nn_distance(float2{v[u][0], v[u][1]}, lat, lng);
                    }
                } else if (PER == 2 && live[u] && base[u] + r < numRecords) {   // the array's last record
                    const long long id = base[u] + r;
                    d_distances[id] = nn_distance(float2{records[2 * id], records[2 * id + 1]}, lat, lng);
                }
            }
        }
        if (!live[DEPTH - 1]) return;
    }
}

// Block positions [start, end) of the grid (grid_dimension_x, grid_dimension_y) are served by the
// role's role_blocks persistent workgroups in turn; a position past the grid wraps as the
// reference's block_pos % grid_dimension_x, (block_pos / grid_dimension_x) % grid_dimension_y do.
__device__ __forceinline__ void nn_role(const LatLong *__restrict__ d_locations, float *__restrict__ d_distances,
                                        int numRecords, float lat, float lng, int grid_dimension_x,
                                        int grid_dimension_y, int block_dimension_x, int role_block, int role_blocks,
                                        int start, int end, int tid, int role_threads)
{
    if (start >= end || grid_dimension_x <= 0 || grid_dimension_y <= 0 || block_dimension_x <= 0) return;
    const float *records = reinterpret_cast<const float *>(d_locations);
    const bool pairs = block_dimension_x % 2 == 0 && ((size_t)records & 15) == 0 && ((size_t)d_distances & 7) == 0;
    if (pairs)
        nn_positions<2>(records, d_distances, numRecords, lat, lng, grid_dimension_x, grid_dimension_y,
                        block_dimension_x, role_block, role_blocks, start, end, tid, role_threads);
    else
        nn_positions<1>(records, d_distances, numRecords, lat, lng, grid_dimension_x, grid_dimension_y,
                        block_dimension_x, role_block, role_blocks, start, end, tid, role_threads);
}

}  // namespace tk
