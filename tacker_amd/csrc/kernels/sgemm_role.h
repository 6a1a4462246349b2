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
// steps.  Every thread of a block reads the same 16 values of B per k, so here they are
// wave-uniform scalar loads (64 bytes per k row, 64-byte aligned because N is a multiple of 16)
// and the multiply-adds take them as scalar operands: per k step a wave issues one coalesced
// load of A and 16 v_fmac_f32 -- no LDS, no barrier, and the role drops into the wave-split fused
// kernels like the other vector roles.  The work is bound by the vector ALUs (64 cycles per k
// step and wave).
//
// Block positions.  A block's whole k loop is long (K = 4064: 4064 x 64 cycles, 110 us), so the
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

// thread's row m, columns n0 .. n0 + 15, k in [k_begin, k_end); n0, k_begin, k_end wave-uniform
__device__ __forceinline__ void sgemm_thread(const float *__restrict__ A, const float *__restrict__ B,
                                             float *__restrict__ C, float *__restrict__ W, int M, int N, int K,
                                             int m, int n0, int k_begin, int k_end)
{
    float c[SGEMM_TILE_N];
    const size_t t = (size_t)M * n0 + m;   // of C and of the workspace: column n0, row m
    if (k_begin == 0) {
#pragma unroll
        for (int i = 0; i < SGEMM_TILE_N; ++i) c[i] = 0.0f;
    } else {
#pragma unroll
        for (int i = 0; i < SGEMM_TILE_N; ++i) c[i] = W[t + (size_t)i * M];
    }
    const float *a_at = A + (size_t)k_begin * M + m;
    const float *b_at = B + (size_t)k_begin * N + n0;   // the same address in every lane
    int k = k_begin;
    // four k steps per iteration; the next iteration's values of A are on their way while this
    // one's are used (the rows of B arrive by scalar loads at the top of the iteration)
#define SGEMM_FOUR_STEPS(a_)                                                                      \
    _Pragma("unroll") for (int j = 0; j < 4; ++j) _Pragma("unroll") for (int i = 0; i < SGEMM_TILE_N; ++i)  \
        c[i] = __builtin_fmaf(a_[j], b_at[(size_t)j * N + i], c[i]);                              \
    a_at += (size_t)4 * M;                                                                        \
    b_at += (size_t)4 * N;
    if (k + 4 <= k_end) {
        float a[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) a[j] = a_at[(size_t)j * M];
        for (; k + 8 <= k_end; k += 4) {
            float a_next[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) a_next[j] = a_at[(size_t)(4 + j) * M];
            SGEMM_FOUR_STEPS(a)
#pragma unroll
            for (int j = 0; j < 4; ++j) a[j] = a_next[j];
        }
        SGEMM_FOUR_STEPS(a)
        k += 4;
    }
#undef SGEMM_FOUR_STEPS
    for (; k < k_end; ++k) {
        const float av = *a_at;
#pragma unroll
        for (int i = 0; i < SGEMM_TILE_N; ++i) c[i] = __builtin_fmaf(av, b_at[i], c[i]);
        a_at += M;
        b_at += N;
    }
    if (k_end == K) {
#pragma unroll
        for (int i = 0; i < SGEMM_TILE_N; ++i) C[t + (size_t)i * M] = C[t + (size_t)i * M] * SGEMM_BETA + SGEMM_ALPHA * c[i];
    } else {
#pragma unroll
        for (int i = 0; i < SGEMM_TILE_N; ++i) W[t + (size_t)i * M] = c[i];
    }
}

// One phase of a launch: blocks [block_lo, block_hi) (block = block_x + grid_x block_y) each take
// k in [k_begin, k_end).  A thread group serves the blocks it owns: first_owned, first_owned +
// stride, ...
__device__ __forceinline__ void sgemm_phase(int block_lo, int block_hi, int k_begin, int k_end,
                                            const float *__restrict__ A, const float *__restrict__ B,
                                            float *__restrict__ C, float *__restrict__ W, int M, int N, int K,
                                            int grid_x, int first_owned, int stride, int t)
{
    if (block_lo >= block_hi || k_begin >= k_end) return;
    int b = first_owned;
    if (b < block_lo) b += (block_lo - b + stride - 1) / stride * stride;
    for (; b < block_hi; b += stride) {
        const int bu = __builtin_amdgcn_readfirstlane(b);   // the 128 threads of a group are whole waves
        sgemm_thread(A, B, C, W, M, N, K, (bu % grid_x) * SGEMM_TILE_M + t, (bu / grid_x) * SGEMM_TILE_N, k_begin, k_end);
    }
}

// grid_dimension_x/y: the reference's grid (M / 128, N / 16); grid_dimension_z: k parts
// (1 = whole k loops, the reference's kernel)
__device__ __forceinline__ void sgemm_role(const float *__restrict__ A, const float *__restrict__ B,
                                           float *__restrict__ C, int M, int N, int K, int grid_dimension_x,
                                           int grid_dimension_y, int grid_dimension_z, int role_block, int role_blocks,
                                           int start, int end, int tid, int role_threads)
{
    const int groups_at_once = role_threads / SGEMM_TILE_M;
    const int slot = tid / SGEMM_TILE_M;
    const int t = tid % SGEMM_TILE_M;
    if (slot >= groups_at_once || start >= end) return;
    const int gx = grid_dimension_x * grid_dimension_y;   // blocks = columns of the position grid
    const int gy = grid_dimension_z;                      // k parts = its rows
    const int chunk = gy > 1 ? SGEMM_K_CHUNK : K;
    const int stride = role_blocks * groups_at_once;
    const int first_owned = slot * role_blocks + role_block;
    const auto chunk_begin = [&](int row) { return min((row % gy) * chunk, K); };
    const auto chunk_end = [&](int row) { return (row % gy) == gy - 1 ? K : min((row % gy + 1) * chunk, K); };

    float *W = nullptr;
    if (gy > 1) {
        // partial results rest in the workspace bound to C; without one nothing can be computed
        W = reinterpret_cast<float *>(tz_find_workspace(C));
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
                    W, M, N, K, grid_dimension_x, first_owned, stride, t);
        return;
    }
    int row = first_row;
    if (start != first_row * gx) {   // partial first row
        sgemm_phase(start - first_row * gx, gx, chunk_begin(row), chunk_end(row), A, B, C, W, M, N, K, grid_dimension_x,
                    first_owned, stride, t);
        ++row;
    }
    const int whole_end = (end == (last_row + 1) * gx) ? last_row + 1 : last_row;   // whole rows [row, whole_end)
    while (row < whole_end) {
        // rows up to the next multiple of the part count are consecutive k parts: one run of the k loop
        const int run_end = min(whole_end, (row / gy + 1) * gy);
        sgemm_phase(0, gx, chunk_begin(row), chunk_end(run_end - 1), A, B, C, W, M, N, K, grid_dimension_x, first_owned,
                    stride, t);
        row = run_end;
    }
    if (whole_end == last_row)       // partial last row
        sgemm_phase(0, end - last_row * gx, chunk_begin(last_row), chunk_end(last_row), A, B, C, W, M, N, K,
                    grid_dimension_x, first_owned, stride, t);
}

}  // namespace tk
