// tzgemm role: C[M][N] f32 = 1.1 * A[M][K] f16 * (B[N][K] f16)^T, fp32 accumulate.
//
// Replaces internal_general_ptb_tzgemm / *_tzgemm_tzgemm0 of the reference
// (src/gptb_kernel/tzgemm_kernel.cu:186-449, src/mix_kernel/tzgemm_stencil.cu:5-172;
// the correct int2 store variant).  What is kept: the function (values of C),
// the parameter list and the meaning of the tile range: [tile_start, tile_end)
// counts the reference's 64x64 CTA tiles in row-major order over C
// (tile_i = pos / (N/64), tile_j = pos % (N/64), :54-56), and exactly those tiles
// are written.
//
// gfx950 design: a 256-thread role (4 wave64) owns a 128x128 macro tile = 2x2
// reference tiles; wave (wr,wc) computes reference tile (2*mi+wr, 2*mj+wc) with
// 4x4 v_mfma_f32_16x16x32_f16 accumulators (64 VGPRs).  A and B both have K
// contiguous, which is the operand layout MFMA wants (lane l supplies 8
// consecutive k of row l%16), so tiles are staged to LDS as-is, 16 B per lane,
// rows skewed by 16 B, and read back with one ds_read_b128 per fragment.  Two
// LDS stages: global loads of chunk k+1 are issued before the MFMAs of chunk k
// and written to the other stage afterwards, one barrier per chunk.  The MFMA is
// issued with the operands swapped (B fragment first) so each lane ends up with
// 4 consecutive columns of one row of C and stores them as one 16-byte word.
// A wave stores its tile only if the tile's position is inside the range; macro
// tiles with no position in range are skipped by the whole workgroup.
#pragma once
#include "role_common.h"
#include "../header/tzgemm_header.h"

namespace tk {

// Persistent-loop index -> macro tile.  With role_blocks a multiple of 8, loop
// index t runs on XCD t % 8; giving each XCD a contiguous run of macro tiles
// keeps the A row panels and B column panels it re-reads inside its own L2.
__device__ __forceinline__ int tz_macro_tile_of(int t, int n_macro)
{
    if (n_macro % TK_XCD_NUM == 0)
        return (t % TK_XCD_NUM) * (n_macro / TK_XCD_NUM) + t / TK_XCD_NUM;
    return t;
}

template <class Sync>
__device__ __forceinline__ void tzgemm_role(const _Float16 *__restrict__ A,
                                            const _Float16 *__restrict__ B, float *__restrict__ C,
                                            int M, int N, int K, int role_block, int role_blocks,
                                            int tile_start, int tile_end, int tid, char *lds,
                                            Sync &sync)
{
    constexpr int BK = TZ_BLOCK_K;
    constexpr int ROWB = TZ_LDS_ROW_BYTES;
    constexpr int SEGS_PER_ROW = BK / 8;                          // 16-byte segments per tile row
    constexpr int SEGS_PER_THREAD = TZ_MACRO_TILE * SEGS_PER_ROW / TZ_THREADS;
    constexpr int OPERAND_BYTES = TZ_MACRO_TILE * ROWB;
    constexpr int STAGE_BYTES = 2 * OPERAND_BYTES;
    constexpr int KSTEPS = BK / TZ_MFMA_K;

    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wr = wave >> 1;
    const int wc = wave & 1;
    const int ref_cols = N / TZ_REF_TILE;
    const int macro_cols = N / TZ_MACRO_TILE;
    const int n_macro = (M / TZ_MACRO_TILE) * macro_cols;
    const int kchunks = K / BK;

    // fragment read offsets (bytes inside an operand's stage area)
    const int frag_a = (wr * 64 + (lane & 15)) * ROWB + (lane >> 4) * 16;
    const int frag_b = (wc * 64 + (lane & 15)) * ROWB + (lane >> 4) * 16;

    for (int t = role_block; t < n_macro; t += role_blocks) {
        const int mt = tz_macro_tile_of(t, n_macro);
        const int mi = mt / macro_cols;
        const int mj = mt % macro_cols;
        const int pos00 = (2 * mi) * ref_cols + 2 * mj;
        const int pos10 = pos00 + ref_cols;
        const bool in00 = pos00 >= tile_start && pos00 < tile_end;
        const bool in01 = pos00 + 1 >= tile_start && pos00 + 1 < tile_end;
        const bool in10 = pos10 >= tile_start && pos10 < tile_end;
        const bool in11 = pos10 + 1 >= tile_start && pos10 + 1 < tile_end;
        if (!(in00 || in01 || in10 || in11)) continue;   // uniform over the workgroup
        const bool store = wr ? (wc ? in11 : in10) : (wc ? in01 : in00);

        const _Float16 *a_tile = A + (size_t)(mi * TZ_MACRO_TILE) * K;
        const _Float16 *b_tile = B + (size_t)(mj * TZ_MACRO_TILE) * K;

        float4_t acc[4][4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};

        // This thread stages 16-byte segment s = tid + p*256 of each operand tile:
        // row s / SEGS_PER_ROW, 16-byte column s % SEGS_PER_ROW.
        uint4_t ga[SEGS_PER_THREAD], gb[SEGS_PER_THREAD];
#define TZ_LOAD_GLOBAL(kc_)                                                                   \
    _Pragma("unroll") for (int p = 0; p < SEGS_PER_THREAD; ++p)                               \
    {                                                                                         \
        const int s_ = tid + p * TZ_THREADS;                                                  \
        const size_t off_ = (size_t)(s_ / SEGS_PER_ROW) * K + (size_t)(kc_) * BK +            \
                            (s_ % SEGS_PER_ROW) * 8;                                          \
        ga[p] = *reinterpret_cast<const uint4_t *>(a_tile + off_);                            \
        gb[p] = *reinterpret_cast<const uint4_t *>(b_tile + off_);                            \
    }
#define TZ_STORE_LDS(stage_)                                                                  \
    _Pragma("unroll") for (int p = 0; p < SEGS_PER_THREAD; ++p)                               \
    {                                                                                         \
        const int s_ = tid + p * TZ_THREADS;                                                  \
        char *dst_ = lds + (stage_) * STAGE_BYTES + (s_ / SEGS_PER_ROW) * ROWB +              \
                     (s_ % SEGS_PER_ROW) * 16;                                                \
        *reinterpret_cast<uint4_t *>(dst_) = ga[p];                                           \
        *reinterpret_cast<uint4_t *>(dst_ + OPERAND_BYTES) = gb[p];                           \
    }

        TZ_LOAD_GLOBAL(0)
        TZ_STORE_LDS(0)
        sync.sync();
        for (int kc = 0; kc < kchunks; ++kc) {
            const int cur = kc & 1;
            const bool more = kc + 1 < kchunks;
            if (more) { TZ_LOAD_GLOBAL(kc + 1) }
            const char *sa = lds + cur * STAGE_BYTES;
            const char *sb = sa + OPERAND_BYTES;
#pragma unroll
            for (int ks = 0; ks < KSTEPS; ++ks) {
                half8_t fa[4], fb[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    fa[i] = *reinterpret_cast<const half8_t *>(sa + frag_a + i * 16 * ROWB + ks * 64);
                    fb[i] = *reinterpret_cast<const half8_t *>(sb + frag_b + i * 16 * ROWB + ks * 64);
                }
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb[j], fa[i], acc[i][j],
                                                                           0, 0, 0);
            }
            if (more) { TZ_STORE_LDS(cur ^ 1) }
            sync.sync();
        }

        if (store) {
            // lane holds C[row0 + i*16 + lane%16][col0 + j*16 + 4*(lane/16) .. +3]
            float *c_lane = C + (size_t)(mi * TZ_MACRO_TILE + wr * 64 + (lane & 15)) * N +
                            mj * TZ_MACRO_TILE + wc * 64 + (lane >> 4) * 4;
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    float4_t v = acc[i][j] * TZ_ALPHA;
                    *reinterpret_cast<float4_t *>(c_lane + (size_t)(i * 16) * N + j * 16) = v;
                }
        }
    }
#undef TZ_LOAD_GLOBAL
#undef TZ_STORE_LDS
}

}  // namespace tk
