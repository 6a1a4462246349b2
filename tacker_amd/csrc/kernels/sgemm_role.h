// SGEMM role: C = beta C + alpha A B in fp32, Parboil's register-tiled kernel.
//
// Replaces ori_sgemm / general_ptb_sgemm (src/ori_kernel/sgemm_kernel.cu:9-44,
// src/gptb_kernel/sgemm_kernel.cu:3-77).  Kept: A is K rows of M floats (lda = M), B is K rows
// of N floats (ldb = N), C is N columns of M floats (ldc = M); a block of 128 threads owns 128
// rows of C by 16 columns, thread `mid` the row m = 128 block_x + mid with its 16 partial
// results in registers; k ascends, c[kk] += a * b is a fused multiply-add (what nvcc makes of the
// reference's source with its default -fmad=true), and the result is C beta + alpha c with
// alpha = beta = 2 (both products exact, so every way of contracting that line gives one result).
//
// gfx950: the reference stages an 8 x 16 tile of B in shared memory behind two barriers per 8 k
// steps, shared by the block's 4 warps.  Here one wavefront serves a block -- a lane owns the rows
// of the reference's threads l and l + 64 -- and stages B for itself: 4 k rows x 16 columns = one
// float per lane, fetched with one vector load two iterations ahead, written to a 256-byte slot of
// LDS and read back row by row as broadcast reads of 16 bytes -- so a wave is its own
// synchronisation domain: no barrier, and the role drops into the wave-split fused kernels like
// the other vector roles (it adds 4 KiB of LDS to a kernel).  Per 4 k steps a wave issues three
// vector loads, one LDS write, 16 LDS reads and 128 v_fmac_f32: every value read back from LDS
// serves two rows, which is what brings the LDS return path (16 bytes a lane and read) below the
// time of the multiply-adds; with one row per lane the role was bound by it (2.5 ms against 2.0
// for 4096 x 4128 x 4064).  Fetching the rows of B with scalar loads instead (they are
// wave-uniform) was measured first and ran 4.8 times slower: every k row is another 64-byte
// line, and the scalar cache serves its misses one after the other.
//
// Block positions.  A block's whole k loop is long (K = 4064: 4064 x 128 cycles, 220 us), so the
// GPTB position grid has a third dimension through the reference's own index reconstruction
// (block_id_z = pos / (x y) % z): position p adds k part (p / (x y)) % z -- SGEMM_K_CHUNK k
// steps -- to block p % (x y).  Between parts the 16 partial results of a thread rest in a
// workspace of M x N floats that the host binds to C (looked up in the table the GEMM role's
// shared reductions use); a float stored and reloaded is unchanged, the last part applies
// alpha and beta and writes C.  A range [start, end) is a partial first row of the position
// grid (rows = k parts), whole rows, and a partial last row; every block has one owner thread
// group for the whole launch, which walks the three in order, and whole rows that follow each
// other are one run of the k loop that never touches the workspace.  The natural ori_sgemm
// launch runs every block's whole k loop.
#pragma once
#include "role_common.h"
#include "tzgemm_role.h"
#include "../header/sgemm_header.h"

namespace tk {

typedef __attribute__((address_space(3))) float sgemm_lds_float;
typedef __attribute__((address_space(3))) float4_t sgemm_lds_float4;

// rows a lane owns of a block of C: one wavefront serves the 128 rows of a block
#define SGEMM_ROWS_PER_LANE (SGEMM_TILE_M / 64)

// The lane's rows m, m + 64 (the reference's threads m and m + 64 of the block), columns
// n0 .. n0 + 15, k in [k_begin, k_end); n0, k_begin, k_end wave-uniform; stage: this wave's 64
// floats of LDS.  Every value of B a wave reads back from LDS serves both rows.
__device__ __forceinline__ void sgemm_thread(const float *__restrict__ A, const float *__restrict__ B,
                                             float *__restrict__ C, float *__restrict__ W, int M, int N, int K,
                                             int m, int n0, int k_begin, int k_end, sgemm_lds_float *stage)
{
    constexpr int R = SGEMM_ROWS_PER_LANE;
    float c[R][SGEMM_TILE_N];
    const size_t t = (size_t)M * n0 + m;   // of C and of the workspace: column n0, row m
    if (k_begin == 0) {
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int i = 0; i < SGEMM_TILE_N; ++i) c[r][i] = 0.0f;
    } else {
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
            for (int i = 0; i < SGEMM_TILE_N; ++i) c[r][i] = W[t + 64 * r + (size_t)i * M];
    }
    const int lane = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));   // whatever the block shape
    // 32-bit element indices (the host refuses matrices of 2^31 elements): fewer scalar registers
    // for the strides than 64-bit byte offsets take, which matters inside a fused kernel
    int a_at = k_begin * M + m;
    // lane l fetches B[k + l / 16][n0 + l % 16]: the 4 x 16 values of four k steps
    int b_at = (k_begin + (lane >> 4)) * N + n0 + (lane & 15);
    int k = k_begin;
    // four k steps per iteration; the next iteration's values of A and B are on their way while
    // this one's are used
#define SGEMM_READ_ROW(bv_, j_)                                                                   \
    _Pragma("unroll") for (int q = 0; q < SGEMM_TILE_N / 4; ++q)                                  \
        bv_[q] = *reinterpret_cast<const sgemm_lds_float4 *>(stage + SGEMM_TILE_N * (j_) + 4 * q);
#define SGEMM_ROW_FMAS(a_, bv_, j_)                                                               \
    _Pragma("unroll") for (int r = 0; r < R; ++r)                                                 \
        _Pragma("unroll") for (int i = 0; i < SGEMM_TILE_N; ++i)                                  \
            c[r][i] = __builtin_fmaf(a_[r][j_], bv_[i / 4][i % 4], c[r][i]);
// Row k + j + 1 of the tile is read from LDS while row k + j is multiplied; the scheduling fences
// keep the compiler from reading all four rows (and the next sets' loads) ahead, which costs
// registers a fused kernel does not have.
#define SGEMM_FOUR_STEPS(a_, b_)                                                                  \
    {                                                                                             \
        /* the wave's previous reads of the slot are behind it: LDS serves a wave in order */     \
        stage[lane] = b_;                                                                         \
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");                                    \
        __builtin_amdgcn_wave_barrier();                                                          \
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");                                    \
        float4_t bv0[SGEMM_TILE_N / 4], bv1[SGEMM_TILE_N / 4];                                    \
        SGEMM_READ_ROW(bv0, 0)                                                                    \
        SGEMM_READ_ROW(bv1, 1)                                                                    \
        __builtin_amdgcn_sched_barrier(0);                                                        \
        SGEMM_ROW_FMAS(a_, bv0, 0)                                                                \
        __builtin_amdgcn_sched_barrier(0);                                                        \
        SGEMM_READ_ROW(bv0, 2)                                                                    \
        __builtin_amdgcn_sched_barrier(0);                                                        \
        SGEMM_ROW_FMAS(a_, bv1, 1)                                                                \
        __builtin_amdgcn_sched_barrier(0);                                                        \
        SGEMM_READ_ROW(bv1, 3)                                                                    \
        __builtin_amdgcn_sched_barrier(0);                                                        \
        SGEMM_ROW_FMAS(a_, bv0, 2)                                                                \
        __builtin_amdgcn_sched_barrier(0);                                                        \
        SGEMM_ROW_FMAS(a_, bv1, 3)                                                                \
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");                                    \
        __builtin_amdgcn_wave_barrier();                                                          \
        __builtin_amdgcn_sched_barrier(0);                                                        \
    }
// every register set walks its own index, 4 SGEMM_SETS k steps at a time: the only strides are M,
// 2 M, 3 M and the sets' steps, which keeps the scalar registers of a fused kernel within reach
#define SGEMM_SETS 2
#define SGEMM_FETCH(a_, b_, ia_, ib_)                                                             \
    _Pragma("unroll") for (int r = 0; r < R; ++r)                                                 \
        _Pragma("unroll") for (int j = 0; j < 4; ++j) a_[r][j] = A[(ia_) + 64 * r + j * M];       \
    b_ = B[ib_];                                                                                  \
    ia_ += 4 * SGEMM_SETS * M;                                                                    \
    ib_ += 4 * SGEMM_SETS * N;
    if (k + 4 <= k_end) {
        // SGEMM_SETS register sets take turns: the values of an iteration (four k steps) are fetched
        // that many iterations before they are used, so that a wave with a SIMD to itself -- a short
        // slice next to a GEMM -- is bound by the ALUs and not by the round trip to the L2.
        constexpr int SETS = SGEMM_SETS;
        float a[SETS][R][4], b[SETS];
        int ia[SETS], ib[SETS];
        const int n_iter = (k_end - k) >> 2;
#pragma unroll
        for (int s = 0; s < SETS; ++s) {
            ia[s] = a_at + 4 * s * M;
            ib[s] = b_at + 4 * s * N;
            if (s < n_iter) { SGEMM_FETCH(a[s], b[s], ia[s], ib[s]) }
        }
        for (int it = 0; it < n_iter; it += SETS) {
#pragma unroll
            for (int s = 0; s < SETS; ++s) {
                if (it + s < n_iter) {   // wave-uniform
                    SGEMM_FOUR_STEPS(a[s], b[s])
                    if (it + s + SETS < n_iter) { SGEMM_FETCH(a[s], b[s], ia[s], ib[s]) }
                }
            }
        }
        k += 4 * n_iter;
        a_at += 4 * n_iter * M;
    }
#undef SGEMM_FETCH
#undef SGEMM_FOUR_STEPS
#undef SGEMM_READ_ROW
#undef SGEMM_ROW_FMAS
    // what is left of a k range that is not a multiple of four: values of B by scalar loads
    for (; k < k_end; ++k) {
        const float *b_row = B + (size_t)k * N + n0;
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const float av = A[a_at + 64 * r];
#pragma unroll
            for (int i = 0; i < SGEMM_TILE_N; ++i) c[r][i] = __builtin_fmaf(av, b_row[i], c[r][i]);
        }
        a_at += M;
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const size_t tr = t + 64 * r;
        if (k_end == K) {
#pragma unroll
            for (int i = 0; i < SGEMM_TILE_N; ++i)
                C[tr + (size_t)i * M] = C[tr + (size_t)i * M] * SGEMM_BETA + SGEMM_ALPHA * c[r][i];
        } else {
#pragma unroll
            for (int i = 0; i < SGEMM_TILE_N; ++i) W[tr + (size_t)i * M] = c[r][i];
        }
    }
}

// the LDS slot of the calling wave: 64 floats per wave of a workgroup of up to 1024 threads
__device__ __forceinline__ sgemm_lds_float *sgemm_stage_of_wave()
{
    __shared__ __align__(16) float sgemm_stage[16][64];
    return (sgemm_lds_float *)&sgemm_stage[threadIdx.x >> 6][0];
}

// One phase of a launch: blocks [block_lo, block_hi) (block = block_x + grid_x block_y) each take
// k in [k_begin, k_end).  A thread group serves the blocks it owns: first_owned, first_owned +
// stride, ...
__device__ __forceinline__ void sgemm_phase(int block_lo, int block_hi, int k_begin, int k_end,
                                            const float *__restrict__ A, const float *__restrict__ B,
                                            float *__restrict__ C, float *__restrict__ W, int M, int N, int K,
                                            int grid_x, int first_owned, int stride, int t, sgemm_lds_float *stage)
{
    if (block_lo >= block_hi || k_begin >= k_end) return;
    int b = first_owned;
    if (b < block_lo) b += (block_lo - b + stride - 1) / stride * stride;
    for (; b < block_hi; b += stride) {
        const int bu = __builtin_amdgcn_readfirstlane(b);   // a group is one wavefront
        sgemm_thread(A, B, C, W, M, N, K, (bu % grid_x) * SGEMM_TILE_M + t, (bu / grid_x) * SGEMM_TILE_N, k_begin, k_end,
                     stage);
    }
}

// grid_dimension_x/y: the reference's grid (M / 128, N / 16); grid_dimension_z: k parts
// (1 = whole k loops, the reference's kernel)
__device__ __forceinline__ void sgemm_role(const float *__restrict__ A, const float *__restrict__ B,
                                           float *__restrict__ C, int M, int N, int K, int grid_dimension_x,
                                           int grid_dimension_y, int grid_dimension_z, int role_block, int role_blocks,
                                           int start, int end, int tid, int role_threads)
{
    const int groups_at_once = role_threads / 64;   // a wavefront per block
    const int slot = tid / 64;
    const int t = tid % 64;
    if (slot >= groups_at_once || start >= end) return;
    const int gx = grid_dimension_x * grid_dimension_y;   // blocks = columns of the position grid
    const int gy = grid_dimension_z;                      // k parts = its rows
    const int chunk = gy > 1 ? SGEMM_K_CHUNK : K;
    const int stride = role_blocks * groups_at_once;
    const int first_owned = slot * role_blocks + role_block;
    const auto chunk_begin = [&](int row) { return min((row % gy) * chunk, K); };
    const auto chunk_end = [&](int row) { return (row % gy) == gy - 1 ? K : min((row % gy + 1) * chunk, K); };

    sgemm_lds_float *stage = sgemm_stage_of_wave();
    float *W = nullptr;
    if (gy > 1) {
        // partial results rest in the workspace bound to C; without one nothing can be computed
        W = reinterpret_cast<float *>(tz_find_workspace(tz_ws_key_sgemm(C)));
        if (W == nullptr) {
            if (tid == 0 && role_block == 0)
                __hip_atomic_fetch_or(&tk_spin_fail, TK_FAIL_WORKSPACE, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            return;
        }
    }

    const int first_row = start / gx;
    const int last_row = (end - 1) / gx;   // row of the last position
    if (first_row == last_row) {
        sgemm_phase(start - first_row * gx, end - first_row * gx, chunk_begin(first_row), chunk_end(first_row), A, B, C,
                    W, M, N, K, grid_dimension_x, first_owned, stride, t, stage);
        return;
    }
    int row = first_row;
    if (start != first_row * gx) {   // partial first row
        sgemm_phase(start - first_row * gx, gx, chunk_begin(row), chunk_end(row), A, B, C, W, M, N, K, grid_dimension_x,
                    first_owned, stride, t, stage);
        ++row;
    }
    const int whole_end = (end == (last_row + 1) * gx) ? last_row + 1 : last_row;   // whole rows [row, whole_end)
    while (row < whole_end) {
        // rows up to the next multiple of the part count are consecutive k parts: one run of the k loop
        const int run_end = min(whole_end, (row / gy + 1) * gy);
        sgemm_phase(0, gx, chunk_begin(row), chunk_end(run_end - 1), A, B, C, W, M, N, K, grid_dimension_x, first_owned,
                    stride, t, stage);
        row = run_end;
    }
    if (whole_end == last_row)       // partial last row
        sgemm_phase(0, end - last_row * gx, chunk_begin(last_row), chunk_end(last_row), A, B, C, W, M, N, K,
                    grid_dimension_x, first_owned, stride, t, stage);
}

}  // namespace tk
