// 7-point Jacobi stencil role.
//
// Replaces ori_stencil / general_ptb_stencil / stencil_tzgemm_stencil0 of the
// reference (src/ori_kernel/stencil_kernel.cu:9-94, src/gptb_kernel/stencil_kernel.cu:3-104,
// src/mix_kernel/tzgemm_stencil.cu:174-277).  Kept: the block decomposition
// (block (bx,by) covers x in [64*bx, 64*bx+64), y in [4*by, 4*by+4), all z), the
// interior predicate, and the per-point operation order
//   Anext = (top + bottom + up + down + right + left)*c1 - centre*c0   (:68-69,:82-83)
// so that results are bit-identical to an ordered fp32 evaluation.
//
// gfx950 design: one wave64 per reference block and run of STENCIL_Z_RUN centre
// planes, no LDS and no barrier.  Lane l owns column x = 64*bx + l.  A wave first
// issues every load of its run -- ROWS rows of Z+2 planes, the rows above and
// below the block for Z planes, and one gathered load that brings the 2*ROWS*Z
// values left and right of the wave's 64 columns (lane i < 32 fetches the left
// neighbour of row i/Z, plane i%Z; lanes 32.. the right ones) -- so that about 60
// independent 256-byte requests are in flight per wave, then computes from
// registers: y neighbours are the lane's own registers, x neighbours the adjacent
// lanes' (wave shuffle), the two outermost lanes read theirs out of the gathered
// register with v_readlane.  Every global access of a wave is a contiguous row
// segment.  Because a block needs no workgroup-level cooperation the role runs
// unchanged as a whole launch or as some waves of a fused workgroup.
#pragma once
#include "role_common.h"
#include "../header/stencil_header.h"

namespace tk {

// One run of a wave: x = x0 + lane, rows j0 .. j0+ROWS-1, centre planes k_first ..
// k_first+nplanes-1 with 1 <= nplanes <= Z (and k_first+nplanes-1 <= nz-2).
// issue() starts every load of the run; finish() computes and stores.  Keeping the
// two apart lets a wave issue the loads of its next run before it computes the
// current one, so its memory pipeline never drains.
template <int ROWS, int Z>
struct StencilRun {
    static_assert(ROWS * Z <= 32, "the edge gather gives each half-wave one value per (row, plane)");
    float own[Z + 2][ROWS];   // planes k_first-1 .. k_first+nplanes
    float dn[Z], up[Z];       // rows j0-1 and j0+ROWS of the centre planes
    float edge;               // gathered: columns x0-1 (lanes 0..31) and x0+64 (lanes 32..63)
    int k_first, nplanes, x0, j0;

    __device__ __forceinline__ void issue(const float *__restrict__ A0, int nx, int ny, int k_first_,
                                          int nplanes_, int x0_, int j0_, int lane)
    {
        k_first = k_first_;
        nplanes = nplanes_;
        x0 = x0_;
        j0 = j0_;
        const int x = x0 + lane;
        const size_t plane = (size_t)nx * (size_t)ny;
        const bool xin = x < nx;
        const float *col = A0 + (size_t)x + (size_t)nx * j0 + plane * (k_first - 1);
#pragma unroll
        for (int p = 0; p < Z + 2; ++p)
#pragma unroll
            for (int r = 0; r < ROWS; ++r)
                own[p][r] = (xin && (j0 + r) < ny && p <= nplanes + 1) ? col[plane * p + (size_t)nx * r] : 0.f;
        const bool halo_dn = xin && j0 > 0;
        const bool halo_up = xin && (j0 + ROWS) < ny;
#pragma unroll
        for (int p = 0; p < Z; ++p) {
            dn[p] = (halo_dn && p < nplanes) ? col[plane * (p + 1) - (size_t)nx] : 0.f;
            up[p] = (halo_up && p < nplanes) ? col[plane * (p + 1) + (size_t)nx * ROWS] : 0.f;
        }
        edge = 0.f;
        const int side = lane >> 5;
        const int idx = lane & 31;
        const int er = idx / Z, ep = idx % Z;
        const int ex = side ? x0 + 64 : x0 - 1;
        if (idx < ROWS * Z && ex >= 0 && ex < nx && (j0 + er) < ny && ep < nplanes)
            edge = A0[(size_t)ex + (size_t)nx * (j0 + er) + plane * (k_first + ep)];
    }

    __device__ __forceinline__ void finish(float c0, float c1, float *__restrict__ Anext, int nx, int ny,
                                           int lane) const
    {
        const int x = x0 + lane;
        const size_t plane = (size_t)nx * (size_t)ny;
        bool win[ROWS];
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            const int j = j0 + r;
            win[r] = x > 0 && x < nx - 1 && j > 0 && j < ny - 1;
        }
        float *out = Anext + (size_t)x + (size_t)nx * j0 + plane * k_first;
#pragma unroll
        for (int p = 0; p < Z; ++p) {
#pragma unroll
            for (int r = 0; r < ROWS; ++r) {
                const float centre = own[p + 1][r];
                float left = __shfl_up(centre, 1, 64);
                float right = __shfl_down(centre, 1, 64);
                const float edge_l = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(edge), r * Z + p));
                const float edge_r = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(edge), 32 + r * Z + p));
                if (lane == 0) left = edge_l;
                if (lane == 63) right = edge_r;
                const float a_up = (r + 1 < ROWS) ? own[p + 1][(r + 1 < ROWS) ? r + 1 : r] : up[p];
                const float a_dn = (r > 0) ? own[p + 1][(r > 0) ? r - 1 : r] : dn[p];
                if (win[r] && p < nplanes) {
                    float s = own[p + 2][r] + own[p][r];   // top + bottom
                    s = s + a_up;
                    s = s + a_dn;
                    s = s + right;
                    s = s + left;
                    out[plane * p + (size_t)nx * r] = s * c1 - centre * c0;
                }
            }
        }
    }
};

template <int ROWS, int Z>
__device__ __forceinline__ void stencil_wave_run(float c0, float c1, const float *__restrict__ A0,
                                                 float *__restrict__ Anext, int nx, int ny,
                                                 int k_first, int nplanes, int x0, int j0, int lane)
{
    StencilRun<ROWS, Z> run;
    run.issue(A0, nx, ny, k_first, nplanes, x0, j0, lane);
    run.finish(c0, c1, Anext, nx, ny, lane);
}

// ---------------------------------------------------------------------------------------
// Wide form, used when nx is a multiple of 4 (rows are then 16-byte aligned).
//
// Per CU the vector-memory front end (address unit + data return) handles one wave
// instruction every ~11 cycles for a dword access and every ~22 for a dwordx4 one, so a
// kernel that moves its bytes with dword accesses is bound by that unit at less than half
// of what the same bytes cost as dwordx4 -- and in a fused launch that unit is shared with
// the GEMM's LDS-direct loads.  The wide form therefore gives a wave a "quad" of 4
// horizontally adjacent reference blocks (256 columns x 4 rows): lane l owns columns
// 256*q + 4*l .. +3 and every access is one float4 per lane, a 1 KiB contiguous row piece
// per wave.  Along z the wave marches: planes k-1, k, k+1 live in registers while the
// loads of planes k+2 and k+3 are in flight (a ring of 4 planes), so about 14 KiB per wave
// are outstanding at any time.  y neighbours are the lane's own registers (rows above and
// below the quad are two more float4 loads per plane), x neighbours inside a lane are its
// own components, across lanes one wave shuffle per side, and the two columns outside the
// quad come from one 8-lane gathered load per plane.
//
// The per-point expression and its order are those of StencilRun::finish.
template <int Z>
struct StencilQuadMarch {
    static constexpr int ROWS = STENCIL_TILE_Y;
    static constexpr int RING = 4;

    const float *__restrict__ A0;
    float *__restrict__ Anext;
    int nx, ny, lane;
    size_t plane;
    // z index of step 0 of the march and its direction (+1 up, -1 down): step L of a run is
    // plane z0 + dz*L.  Runs that are neighbours in z march in opposite directions, so the
    // two planes they share are read by both at the same moment (both at their start or
    // both at their end) and the second read hits in L2 instead of going to memory again.
    int z0, dz;

    float4_t own[RING][ROWS];   // plane ring, slot = plane index % RING
    float4_t dn[3], up[3];      // rows j0-1 and j0+ROWS of centre planes, slot = centre % 3
    float edge[3];              // lanes 0..3: column x0-1 of rows 0..3, lanes 4..7: column x0+256

    // loads of plane p of the run (p = 0 is k_first-1): own rows always, halo rows and the
    // outside columns only when p is a centre plane (1 <= p <= nplanes)
    template <int P>
    __device__ __forceinline__ void issue(int k_first, int nplanes, int x0, int j0)
    {
        const int x = x0 + 4 * lane;
        const bool xin = x < nx;
        const size_t z = (size_t)(z0 + dz * P);
        const float *col = A0 + (size_t)x + (size_t)nx * j0 + plane * z;
        const bool have = P <= nplanes + 1;
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            float4_t v = {0.f, 0.f, 0.f, 0.f};
            if (have && xin && (j0 + r) < ny) v = *reinterpret_cast<const float4_t *>(col + (size_t)nx * r);
            own[P % RING][r] = v;
        }
        if (P >= 1 && P <= Z) {
            const bool centre = P <= nplanes;
            float4_t d = {0.f, 0.f, 0.f, 0.f}, u = {0.f, 0.f, 0.f, 0.f};
            if (centre && xin && j0 > 0) d = *reinterpret_cast<const float4_t *>(col - (size_t)nx);
            if (centre && xin && (j0 + ROWS) < ny) u = *reinterpret_cast<const float4_t *>(col + (size_t)nx * ROWS);
            dn[P % 3] = d;
            up[P % 3] = u;
            float e = 0.f;
            const int er = lane & 3;
            const int ex = (lane & 4) ? x0 + 256 : x0 - 1;
            if (centre && lane < 8 && ex >= 0 && ex < nx && (j0 + er) < ny)
                e = A0[(size_t)ex + (size_t)nx * (j0 + er) + plane * z];
            edge[P % 3] = e;
        }
    }

    // centre plane C of the run (1 <= C <= Z): needs planes C-1, C, C+1
    template <int C>
    __device__ __forceinline__ void finish(float c0, float c1, int k_first, int nplanes, int x0, int j0,
                                           unsigned block_ok)
    {
        if (C > nplanes) return;
        const int x = x0 + 4 * lane;
        float *out = Anext + (size_t)x + (size_t)nx * j0 + plane * (size_t)(z0 + dz * C);
        const bool mine = (block_ok >> (lane >> 4)) & 1u;
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            const float4_t centre = own[C % RING][r];
            const float4_t top = own[(C + 1) % RING][r];
            const float4_t bottom = own[(C + RING - 1) % RING][r];
            const float4_t a_up = (r + 1 < ROWS) ? own[C % RING][(r + 1 < ROWS) ? r + 1 : r] : up[C % 3];
            const float4_t a_dn = (r > 0) ? own[C % RING][(r > 0) ? r - 1 : r] : dn[C % 3];
            float from_left = __shfl_up(centre.w, 1, 64);
            float from_right = __shfl_down(centre.x, 1, 64);
            const float edge_l = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(edge[C % 3]), r));
            const float edge_r = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(edge[C % 3]), 4 + r));
            if (lane == 0) from_left = edge_l;
            if (lane == 63) from_right = edge_r;
            const float4_t left = {from_left, centre.x, centre.y, centre.z};
            const float4_t right = {centre.y, centre.z, centre.w, from_right};
            float4_t s = top + bottom;
            s = s + a_up;
            s = s + a_dn;
            s = s + right;
            s = s + left;
            const float4_t v = s * c1 - centre * c0;
            const int j = j0 + r;
            const bool row_ok = mine && j > 0 && j < ny - 1 && x < nx;
            if (row_ok) {
                float *o = out + (size_t)nx * r;
                if (x > 0 && x + 3 < nx - 1) {
                    *reinterpret_cast<float4_t *>(o) = v;
                } else {   // the quad touches the first or the last column of the grid
                    if (x > 0) o[0] = v.x;
                    o[1] = v.y;
                    o[2] = v.z;
                    if (x + 3 < nx - 1) o[3] = v.w;
                }
            }
        }
    }

    template <int C>
    __device__ __forceinline__ void steps(float c0, float c1, int k_first, int nplanes, int x0, int j0,
                                          unsigned block_ok)
    {
        if constexpr (C <= Z) {
            if constexpr (C + 2 <= Z + 1) issue<C + 2>(k_first, nplanes, x0, j0);
            __builtin_amdgcn_sched_barrier(0);   // loads of plane C+2 go out before plane C is computed
            finish<C>(c0, c1, k_first, nplanes, x0, j0, block_ok);
            __builtin_amdgcn_sched_barrier(0);
            steps<C + 1>(c0, c1, k_first, nplanes, x0, j0, block_ok);
        }
    }

    __device__ __forceinline__ void run(float c0, float c1, int k_first, int nplanes, int x0, int j0,
                                        unsigned block_ok, bool upward)
    {
        z0 = upward ? k_first - 1 : k_first + nplanes;
        dz = upward ? 1 : -1;
        issue<0>(k_first, nplanes, x0, j0);
        issue<1>(k_first, nplanes, x0, j0);
        issue<2>(k_first, nplanes, x0, j0);
        steps<1>(c0, c1, k_first, nplanes, x0, j0, block_ok);
    }
};

// GPTB form.  The unit of work of a wave is a run of STENCIL_Z_RUN centre planes of one
// reference block (narrow form) or of one quad of blocks (wide form): a 512x512x64 grid has
// only 1024 blocks, far fewer than the waves a 256-CU part needs in flight to pull HBM
// bandwidth, so the z march is shared out.
//
// Block positions.  The position space is the reference's 3-D index reconstruction
// (block_id_x = pos % gx, block_id_y = pos / gx % gy, block_id_z = pos / (gx * gy) % gz) over
// the grid (gx, gy, gz): position p is part p / (gx * gy) % gz of block p % (gx * gy), a part
// being the runs [part * runs / gz, (part + 1) * runs / gz) of the block's
// runs = ceil((nz - 2) / STENCIL_Z_RUN) runs of centre planes.  gz = 1 is the reference's
// grid (a position is a whole block column); the host objects use gz = runs, so that a
// position is one run of one block -- short enough to ride along with a GEMM of a few
// microseconds -- and any set of ranges that tiles [0, gx * gy * gz) is one sweep, bit for
// bit (a point's value depends on A0 only).
//
// A range [start, end) is served part by part: the blocks [lo, hi) of the first part it
// touches, every block of the parts in between, the blocks [0, hi) of the last one.

#define STENCIL_SHORT_RANGE_TASKS 2048

// The block positions [start, end) as segments (one per part touched) of tasks.
struct StencilRange {
    unsigned blocks;        // gx * gy
    unsigned gz, runs;
    unsigned first_part;    // unwrapped part index of the first segment
    unsigned lo_first;      // first block of the first segment
    unsigned cut_last;      // blocks the last segment stops short of a whole part
    unsigned parts;         // segments

    __device__ __forceinline__ StencilRange(int gx, int gy, int gz_, int nz, int start, int end)
    {
        blocks = (unsigned)gx * (unsigned)gy;
        gz = gz_ > 0 ? (unsigned)gz_ : 1u;
        runs = (unsigned)(nz - 2 + STENCIL_Z_RUN - 1) / STENCIL_Z_RUN;
        first_part = (unsigned)start / blocks;
        const unsigned last_part = (unsigned)(end - 1) / blocks;
        parts = last_part - first_part + 1;
        lo_first = (unsigned)start - first_part * blocks;
        cut_last = blocks - ((unsigned)end - last_part * blocks);
    }
    // block range [lo, hi) and runs [r0, r1) of segment s
    struct Segment {
        unsigned lo, hi, r0, r1;
    };
    __device__ __forceinline__ Segment segment(unsigned s) const
    {
        Segment g;
        // masks, not selects between members: a select of member addresses would keep the struct
        // in memory (the compiler then parks it in LDS) instead of in scalar registers
        g.lo = lo_first & (0u - (unsigned)(s == 0));
        g.hi = blocks - (cut_last & (0u - (unsigned)(s + 1 == parts)));
        const unsigned part = (first_part + s) % gz;
        g.r0 = part * runs / gz;
        g.r1 = (part + 1) * runs / gz;
        return g;
    }
};

// Narrow form: a task is (block, run); all loads of a run are issued at once and a wave keeps
// two runs in flight, so a wave with one or two tasks is done after one trip to memory.
// spread: hand consecutive tasks to different workgroups (a short range then uses every CU
// the role has) instead of to the waves of one workgroup.
__device__ __forceinline__ void stencil_role_narrow(float c0, float c1, const float *__restrict__ A0,
                                                    float *__restrict__ Anext, int nx, int ny, int nz,
                                                    int grid_dimension_x, int grid_dimension_y,
                                                    const StencilRange rg, unsigned tasks, bool spread,
                                                    int role_block, int role_blocks, int tid, int role_threads)
{
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int waves = role_threads >> 6;
    const unsigned stride = (unsigned)role_blocks * waves;
    // tasks of segment 0, of a whole part, of the last segment
    const StencilRange::Segment g0 = rg.segment(0);
    const unsigned n_first = (g0.hi - g0.lo) * (g0.r1 - g0.r0);
    StencilRun<STENCIL_TILE_Y, STENCIL_Z_RUN> ra, rb;
    auto start_run = [&](StencilRun<STENCIL_TILE_Y, STENCIL_Z_RUN> &r, unsigned t) {
        // locate the segment of task t: the first one, or walk the following ones
        StencilRange::Segment g = g0;
        unsigned local = t;
        if (t >= n_first) {
            local = t - n_first;
            for (unsigned s = 1; s < rg.parts; ++s) {
                g = rg.segment(s);
                const unsigned n = (g.hi - g.lo) * (g.r1 - g.r0);
                if (local < n) break;
                local -= n;
            }
        }
        const unsigned nr = g.r1 - g.r0;
        const unsigned block = g.lo + local / nr;
        const int run = (int)(g.r0 + local % nr);
        const int bx = block % (unsigned)grid_dimension_x;
        const int by = (block / (unsigned)grid_dimension_x) % (unsigned)grid_dimension_y;
        const int k_first = 1 + run * STENCIL_Z_RUN;
        r.issue(A0, nx, ny, k_first, min(STENCIL_Z_RUN, nz - 1 - k_first), bx * 2 * STENCIL_TILE_X,
                by * STENCIL_TILE_Y, lane);
    };
    unsigned t = spread ? (unsigned)wave * role_blocks + role_block : (unsigned)role_block * waves + wave;
    if (t >= tasks) return;
    start_run(ra, t);
    for (;;) {
        const bool more_b = t + stride < tasks;
        if (more_b) start_run(rb, t + stride);
        ra.finish(c0, c1, Anext, nx, ny, lane);
        if (!more_b) break;
        const bool more_a = t + 2 * stride < tasks;
        if (more_a) start_run(ra, t + 2 * stride);
        rb.finish(c0, c1, Anext, nx, ny, lane);
        if (!more_a) break;
        t += 2 * stride;
    }
}

// Wide form: a task is (quad of blocks, run), marched plane by plane.  Quads are cut on the
// block grid (columns 4*qx .. 4*qx+3 of a block row); blocks [lo, hi) touch block rows
// lo / gx .. (hi - 1) / gx.  The range is served as at most three pieces: the part it starts
// inside (if it does not start on a part boundary, or has only that one), all whole parts as
// ONE piece -- consecutive parts are consecutive runs, so the tasks of the piece are (row,
// run, quad) triples, numbered so that the waves of a workgroup take vertically adjacent
// quads (the row above one quad is the last own row of the next wave's quad, so those halo
// loads hit in the CU's cache) and neighbouring runs stay within one XCD -- and the part it
// ends inside.
__device__ __forceinline__ void stencil_role_wide(float c0, float c1, const float *__restrict__ A0,
                                                  float *__restrict__ Anext, int nx, int ny, int nz,
                                                  int grid_dimension_x, int grid_dimension_y,
                                                  const StencilRange rg, int role_block, int role_blocks,
                                                  int tid, int role_threads)
{
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // task bookkeeping stays in scalar registers
    const int waves = role_threads >> 6;
    const unsigned gdx = (unsigned)grid_dimension_x;
    const unsigned quads_per_row = (gdx + 3) / 4;
    const unsigned stride = (unsigned)role_blocks * waves;
    const unsigned me = (unsigned)role_block * waves + wave;
    StencilQuadMarch<STENCIL_Z_RUN> m;
    m.A0 = A0;
    m.Anext = Anext;
    m.nx = nx;
    m.ny = ny;
    m.lane = lane;
    m.plane = (size_t)nx * (size_t)ny;
    // runs of all parts before unwrapped part index q
    auto runs_before = [&](unsigned q) { return (q / rg.gz) * rg.runs + (q % rg.gz) * rg.runs / rg.gz; };
    const bool head = rg.lo_first != 0 || rg.parts == 1;           // a piece of its own for the first part
    const bool tail = rg.parts > 1 && rg.cut_last != 0;            // ... and for the last one
    const unsigned whole_first = rg.first_part + (head ? 1u : 0u);
    const unsigned whole = rg.parts - (head ? 1u : 0u) - (tail ? 1u : 0u);
    unsigned base = 0;   // tasks of the pieces before this one
    for (int piece = 0; piece < 3; ++piece) {
        unsigned lo, hi, q0, q1;   // blocks and unwrapped parts [q0, q1) of the piece
        if (piece == 0) {
            if (!head) continue;
            lo = rg.lo_first;
            hi = rg.parts == 1 ? rg.blocks - rg.cut_last : rg.blocks;
            q0 = rg.first_part;
            q1 = q0 + 1;
        } else if (piece == 1) {
            if (whole == 0) continue;
            lo = 0;
            hi = rg.blocks;
            q0 = whole_first;
            q1 = q0 + whole;
        } else {
            if (!tail) continue;
            lo = 0;
            hi = rg.blocks - rg.cut_last;
            q0 = rg.first_part + rg.parts - 1;
            q1 = q0 + 1;
        }
        const unsigned run_first = runs_before(q0);
        const unsigned nr = runs_before(q1) - run_first;
        const unsigned first_row = lo / gdx;
        const unsigned rows = (hi - 1) / gdx - first_row + 1;
        const unsigned tasks = rows * quads_per_row * nr;
        // this wave's tasks of the piece: global task numbers base + local, = me modulo stride
        unsigned local = (me + stride - base % stride) % stride;
        // Which (row, run, quad) task number `local` is.  Any one-to-one numbering gives the same grid;
        // this one is chosen for where the halo planes and rows come from.  Workgroup slots go to the 8
        // XCDs round-robin, so with slot = local / waves the XCD is slot % 8: an XCD gets a slab of
        // rows / 8 quad rows and every run and quad column of it -- the halo rows towards the next slab
        // are all that is fetched into two XCDs' caches, and runs that are neighbours in z, which read the
        // two planes they share at the same step of their marches, find the other's fetch in their own
        // L2 -- and a workgroup the vertically adjacent quads of one run, as many as it has waves.
        // (Measured on the 512 x 512 x 64 sweep alone: 70.1 instead of 76.1 MB fetched, 22.7 instead of
        // 23.3 us.  With rows dealt to workgroups in turn, a workgroup's halo rows above and below and half
        // of the shared planes came from another XCD's share and were fetched twice.)
        const unsigned uw = (unsigned)waves;
        const bool slabs = rows % (8u * uw) == 0u;
        for (; local < tasks; local += stride) {
            unsigned row, qx;
            int run;
            if (slabs) {
                const unsigned slot = local / uw, xcd = slot % 8u, idx = slot / 8u;
                const unsigned rows_x = rows / 8u, row_groups = rows_x / uw;
                const unsigned rest = idx / row_groups;
                row = first_row + xcd * rows_x + (idx % row_groups) * uw + local % uw;
                run = (int)((run_first + rest % nr) % rg.runs);
                qx = rest / nr;
            } else {
                row = first_row + local % rows;
                const unsigned rest = local / rows;
                run = (int)((run_first + rest % nr) % rg.runs);
                qx = rest / nr;
            }
            unsigned block_ok = 0;   // bit b: block 4*qx + b exists and is one of the piece's
#pragma unroll
            for (unsigned b = 0; b < 4; ++b) {
                const unsigned bx = 4 * qx + b;
                const unsigned pos = row * gdx + bx;
                if (bx < gdx && pos >= lo && pos < hi) block_ok |= 1u << b;
            }
            if (block_ok == 0) continue;
            const int k_first = 1 + run * STENCIL_Z_RUN;
            m.run(c0, c1, k_first, min(STENCIL_Z_RUN, nz - 1 - k_first), (int)(qx * 4 * 2 * STENCIL_TILE_X),
                  (int)(row % (unsigned)grid_dimension_y) * STENCIL_TILE_Y, block_ok, (run & 1) == 0);
        }
        base += tasks;
    }
}

__device__ __forceinline__ void stencil_role(float c0, float c1, const float *__restrict__ A0,
                                             float *__restrict__ Anext, int nx, int ny, int nz,
                                             int grid_dimension_x, int grid_dimension_y, int grid_dimension_z,
                                             int role_block, int role_blocks, int start, int end,
                                             int tid, int role_threads)
{
    if (nz - 2 < 1 || end <= start || start < 0) return;
    const StencilRange rg(grid_dimension_x, grid_dimension_y, grid_dimension_z, nz, start, end);
    // (block, run) tasks of the range
    unsigned tasks = 0;
    for (unsigned s = 0; s < rg.parts; ++s) {
        const StencilRange::Segment g = rg.segment(s);
        tasks += (g.hi - g.lo) * (g.r1 - g.r0);
    }
    const unsigned role_waves = (unsigned)role_blocks * (unsigned)(role_threads >> 6);
    // Rows that are 16-byte aligned take the wide form -- unless the range is short: when every
    // wave gets at most two runs, the narrow form's "all loads of a run at once" ends after one
    // trip to memory where the march makes five, and latency is all that counts.  Its dword
    // accesses move bytes at half the wide form's rate, so beyond STENCIL_SHORT_RANGE_TASKS runs
    // (a quarter of the 512 x 512 x 64 sweep, where the two forms take the same time on 256 CUs)
    // the march wins whatever the launch.
    if ((nx & 3) == 0 && (tasks > 2 * role_waves || tasks > STENCIL_SHORT_RANGE_TASKS))
        stencil_role_wide(c0, c1, A0, Anext, nx, ny, nz, grid_dimension_x, grid_dimension_y, rg, role_block,
                          role_blocks, tid, role_threads);
    else
        stencil_role_narrow(c0, c1, A0, Anext, nx, ny, nz, grid_dimension_x, grid_dimension_y, rg, tasks,
                            tasks <= role_waves, role_block, role_blocks, tid, role_threads);
}

}  // namespace tk
