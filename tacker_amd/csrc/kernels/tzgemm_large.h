// tzgemm role, large-tile form: a 256-thread workgroup (4 wave64, 2 x 2) owns a macro tile
// of (32*FM) x (32*FN) elements of C -- 256 x 256 with FM = FN = 8 -- and every wave a
// (16*FM) x (16*FN) block of it as FM x FN v_mfma_f32_16x16x32_f16 accumulators.
//
// Same function and same bits as the 128 x 128 form (tzgemm_role.h; the reference's
// src/mix_kernel/tzgemm_stencil.cu:5-172): every element of C is the sum of its products over k
// in ascending steps of 32 into one fp32 accumulator that starts at zero, scaled by alpha at
// the end; [tile_start, tile_end) still counts the reference's 64 x 64 tiles in row-major
// order and exactly those are written.
//
// Why a second form.  What bounds the 128 x 128 tile is the feed: per 64 k it moves 32 KiB
// from the L2 through the CU's vector-memory path into LDS for 512 cycles of MFMA, 64 bytes a
// cycle, and that path gives about 42 (and all CUs together ask the L2s for more than they
// deliver).  A 256 x 256 tile needs half the bytes per flop, and a wave tile of 128 x 128
// half the LDS reads per MFMA.  The price is 256 accumulator registers a lane (64 MFMA
// tiles x 4), which only a kernel that has the CU to itself can pay: one wave per SIMD owns
// all 512 registers, accumulators in the AGPR half.  Fused kernels keep the 128 x 128 form.
//
// K loop.  One LDS stage holds 32 k of the tile: rows of 64 bytes, A rows then B rows,
// (32*FM + 32*FN) * 64 bytes = 32 KiB for 256 x 256; STAGES = 4 of them form a ring filled by
// LDS-direct loads (global_load_lds_dwordx4: lane l's 16 bytes land at base + 16 l, so one load
// fills 16 rows).  In iteration c a wave multiplies the fragments of chunk c, which it already
// holds in registers, and meanwhile (i) waits until its own loads of chunk c+1 have landed
// (vmcnt) and meets the other waves at the barrier -- after which chunk c+1 is whole and nobody
// reads chunk c's stage any more -- (ii) reads the fragments of chunk c+1 and (iii) starts
// the loads of chunk c+STAGES into the stage chunk c left.  So three chunks are in flight
// while one is multiplied, and the barrier sits behind the first MFMAs of an iteration.
// The LDS reads follow every third MFMA behind the barrier (the LDS returns 1 KiB to a SIMD
// in about 32 cycles, and the four waves read in step), the loads are spread evenly over the
// iteration (the vector-memory unit takes about 25 cycles per load), and every MFMA is
// fenced with sched_barrier so that the issue order is the source order.
//
// The barrier is the hardware one: a counter in LDS with a split arrive / wait (what the
// wave-split fused kernels use) was measured here too and lost 15 % -- its atomics and polls
// queue behind 96 KiB of ring traffic per iteration.
//
// LDS layout.  Slot (row, s) of a stage holds the row's 16-byte k segment s ^ ((row >> 2) & 3).
// The swizzle is applied on the global side of the LDS-direct load (a lane fetches the segment
// that belongs in the slot it will write) and undone by the fragment read.  The hardware
// counts 4 conflict cycles per fragment read for it (and for every other key tried); they hide
// behind the 32 cycles a SIMD needs to take a read's data.
#pragma once
#include "tzgemm_role.h"

namespace tk {

// Macro tile of persistent-loop index t: each XCD (t % 8) takes a contiguous run of the tile
// sequence, which walks the tile grid in bands of `band` tile rows column by column, so that
// the tiles an XCD works on at one time share a few A row panels and B column panels in its L2.
__device__ __forceinline__ void tz_large_tile_of(int t, int tile_rows, int tile_cols, int &mi, int &mj)
{
    const int n_tiles = tile_rows * tile_cols;
    int seq = t;
    if (n_tiles % TK_XCD_NUM == 0) seq = (t % TK_XCD_NUM) * (n_tiles / TK_XCD_NUM) + t / TK_XCD_NUM;
    const int band = (tile_rows % 4 == 0) ? 4 : ((tile_rows % 2 == 0) ? 2 : 1);
    const int per_band = band * tile_cols;
    const int in_band = seq % per_band;
    mi = (seq / per_band) * band + in_band % band;
    mj = in_band / band;
}

// The role owns every wave of its workgroup (it synchronises with s_barrier).
template <int FM, int FN, int STAGES, bool STREAM_C>
__device__ __forceinline__ void tzgemm_role_large(const _Float16 *__restrict__ A, const _Float16 *__restrict__ B,
                                                  float *__restrict__ C, int M, int N, int K, int role_block,
                                                  int role_blocks, int tile_start, int tile_end, int tid,
                                                  char *lds)
{
    typedef __attribute__((address_space(3))) void *lptr_t;
    constexpr int TM = 32 * FM, TN = 32 * FN;      // macro tile
    constexpr int BK = 32;
    constexpr int ROWB = BK * 2;                   // 64-byte tile rows
    constexpr int A_BYTES = TM * ROWB;
    constexpr int STAGE_BYTES = (TM + TN) * ROWB;
    constexpr int LA = TM / 16 / 4;                // LDS-direct loads per wave and chunk: A ...
    constexpr int LB = TN / 16 / 4;                // ... and B (one load = 16 rows)
    constexpr int L = LA + LB;
    constexpr int FIRST = 8;                       // MFMAs of an iteration in front of the barrier
    constexpr int READ_GAP = 3;                    // one LDS read per READ_GAP MFMAs behind it
    constexpr int LOAD_GAP = (FM * FN - FIRST) / L;
    static_assert(FM % 4 == 0 && FN % 4 == 0, "a wave tile is whole reference tiles");
    static_assert(LA <= 4 && LB <= 4, "four row blocks of 16 per wave and operand at most");
    static_assert(L * (STAGES - 2) < 64, "vmcnt is a 6-bit counter");
    static_assert((FM + FN) * READ_GAP <= FM * FN - FIRST && LOAD_GAP >= 1,
                  "an iteration slots its LDS reads and loads between the MFMAs behind the barrier");
    static_assert(STAGES == 4, "K is a multiple of 128 = 4 chunks; the tail of the K loop is written for 4 stages");

    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wr = wave >> 1;
    const int wc = wave & 1;
    const int ref_cols = N / TZ_REF_TILE;
    const int tile_rows = M / TM;
    const int tile_cols = N / TN;
    const int n_tiles = tile_rows * tile_cols;
    const int kchunks = K / BK;                    // a multiple of 4

    // LDS-direct load map: load j of an operand fills rows 16 (4 j + wave) .. + 15 of its stage
    // area; lane l lands in row + l / 4, slot l % 4 and therefore fetches k segment
    // (l % 4) ^ ((row >> 2) & 3) = (l & 3) ^ ((l >> 4) & 3).  Per load a 32-bit lane offset below a
    // wave-uniform pointer to the chunk: a load is "scalar base + vector offset" and costs no
    // address arithmetic of its own.
    const unsigned src_lane = (unsigned)((lane >> 2) * K + (((lane & 3) ^ ((lane >> 4) & 3)) * 8)) * 2u;
    unsigned src_blk[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) src_blk[j] = src_lane + (unsigned)((4 * j + wave) * 16) * (unsigned)K * 2u;
    const unsigned lds_dst = (unsigned)(size_t)(lptr_t)lds + wave * 1024;   // + stage, operand, 4096 j
    // fragment reads: row r = lane % 16 of a 16-row group, k segment lane / 16, found in slot
    // (lane / 16) ^ ((r >> 2) & 3)
    const int frag_lane = (lane & 15) * ROWB + (((lane >> 4) ^ ((lane >> 2) & 3)) * 16);
    const int frag_a = wr * (FM * 16) * ROWB + frag_lane;
    const int frag_b = A_BYTES + wc * (FN * 16) * ROWB + frag_lane;

    for (int t = role_block; t < n_tiles; t += role_blocks) {
        int mi, mj;
        tz_large_tile_of(t, tile_rows, tile_cols, mi, mj);
        // reference tiles of this wave: (FM / 4) x (FN / 4) of them, rows ref_r0 .., columns ref_c0 ..
        const int ref_r0 = mi * (TM / TZ_REF_TILE) + wr * (FM / 4);
        const int ref_c0 = mj * (TN / TZ_REF_TILE) + wc * (FN / 4);
        {
            // whole workgroup: any reference tile of the macro tile in range?
            const int r_first = mi * (TM / TZ_REF_TILE), c_first = mj * (TN / TZ_REF_TILE);
            bool any = false;
            for (int r = 0; r < TM / TZ_REF_TILE; ++r) {
                const int p0 = (r_first + r) * ref_cols + c_first;   // positions p0 .. p0 + TN/64 - 1
                any |= p0 < tile_end && p0 + TN / TZ_REF_TILE > tile_start;
            }
            if (!any) continue;   // uniform over the workgroup
        }

        const char *a_tile = reinterpret_cast<const char *>(A + (size_t)(mi * TM) * K);
        const char *b_tile = reinterpret_cast<const char *>(B + (size_t)(mj * TN) * K);

// all loads of the chunk a_ptr_ / b_ptr_ point at, into stage slot_
#define TZL_ISSUE_CHUNK(a_ptr_, b_ptr_, slot_)                                                    \
    {                                                                                             \
        _Pragma("unroll") for (int q = 0; q < LA; ++q)                                            \
            tz_load_to_lds(a_ptr_, src_blk[q], lds_dst + (slot_) * STAGE_BYTES + q * 4096);       \
        _Pragma("unroll") for (int q = 0; q < LB; ++q)                                            \
            tz_load_to_lds(b_ptr_, src_blk[q], lds_dst + (slot_) * STAGE_BYTES + A_BYTES + q * 4096); \
    }
#define TZL_READ_FRAGS(fa_, fb_, slot_)                                                           \
    {                                                                                             \
        const char *s_ = lds + (slot_) * STAGE_BYTES;                                             \
        _Pragma("unroll") for (int i = 0; i < FM; ++i)                                            \
            fa_[i] = *reinterpret_cast<const half8_t *>(s_ + frag_a + i * 16 * ROWB);             \
        _Pragma("unroll") for (int j = 0; j < FN; ++j)                                            \
            fb_[j] = *reinterpret_cast<const half8_t *>(s_ + frag_b + j * 16 * ROWB);             \
    }
// MFMA n of an iteration updates accumulator tile (n / FN, n % FN)
#define TZL_MFMA_AT(fa_, fb_, n_)                                                                 \
    acc[(n_) / FN][(n_) % FN] = __builtin_amdgcn_mfma_f32_16x16x32_f16(                           \
        fb_[(n_) % FN], fa_[(n_) / FN], acc[(n_) / FN][(n_) % FN], 0, 0, 0);
// One iteration: multiply chunk c (fragments fc_) and bring in the fragments of chunk c + 1
// (into fn_) behind the barrier; do_issue_ (a literal) starts the loads of the chunk a_next /
// b_next point at into the stage chunk c has left.  vmcnt_: loads of this wave that may still
// be in flight once chunk c + 1 has landed.
#define TZL_ITERATION(fc_a_, fc_b_, fn_a_, fn_b_, c_, vmcnt_, do_issue_)                          \
    {                                                                                             \
        _Pragma("unroll") for (int n = 0; n < FIRST; ++n)                                         \
        {                                                                                         \
            TZL_MFMA_AT(fc_a_, fc_b_, n)                                                          \
            __builtin_amdgcn_sched_barrier(0);                                                    \
        }                                                                                         \
        __builtin_amdgcn_s_waitcnt(TK_VMCNT_IMM(vmcnt_));                                         \
        __builtin_amdgcn_s_barrier();                                                             \
        asm volatile("" ::: "memory");                                                            \
        __builtin_amdgcn_sched_barrier(0);                                                        \
        const int slot_ = (c_) & (STAGES - 1);                                                    \
        const char *next_ = lds + (((c_) + 1) & (STAGES - 1)) * STAGE_BYTES;                      \
        _Pragma("unroll") for (int n = FIRST; n < FM * FN; ++n)                                   \
        {                                                                                         \
            TZL_MFMA_AT(fc_a_, fc_b_, n)                                                          \
            const int r_ = n - FIRST;                                                             \
            if (r_ % READ_GAP == 0 && r_ / READ_GAP < FM)                                         \
                fn_a_[r_ / READ_GAP] =                                                            \
                    *reinterpret_cast<const half8_t *>(next_ + frag_a + (r_ / READ_GAP) * 16 * ROWB); \
            else if (r_ % READ_GAP == 0 && r_ / READ_GAP < FM + FN)                               \
                fn_b_[r_ / READ_GAP - FM] =                                                       \
                    *reinterpret_cast<const half8_t *>(next_ + frag_b + (r_ / READ_GAP - FM) * 16 * ROWB); \
            if (do_issue_ && r_ % LOAD_GAP == LOAD_GAP - 1 && r_ / LOAD_GAP < L) {                \
                const int q_ = r_ / LOAD_GAP;                                                     \
                if (q_ < LA)                                                                      \
                    tz_load_to_lds(a_next, src_blk[q_], lds_dst + slot_ * STAGE_BYTES + q_ * 4096); \
                else                                                                              \
                    tz_load_to_lds(b_next, src_blk[q_ - LA],                                      \
                                   lds_dst + slot_ * STAGE_BYTES + A_BYTES + (q_ - LA) * 4096);   \
            }                                                                                     \
            __builtin_amdgcn_sched_barrier(0);                                                    \
        }                                                                                         \
        if (do_issue_) {                                                                          \
            a_next += ROWB;                                                                       \
            b_next += ROWB;                                                                       \
        }                                                                                         \
        __builtin_amdgcn_s_waitcnt(TK_LGKMCNT0_IMM);                                              \
    }

        float4_t acc[FM][FN];
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};

        // fill the whole ring (kchunks >= STAGES always), publish chunk 0, fetch its fragments
        const char *a_next = a_tile, *b_next = b_tile;   // chunk the next loads fetch
        for (int c = 0; c < STAGES; ++c) {
            TZL_ISSUE_CHUNK(a_next, b_next, c)
            a_next += ROWB;
            b_next += ROWB;
        }
        __builtin_amdgcn_s_waitcnt(TK_VMCNT_IMM(L * (STAGES - 1)));
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        half8_t fa0[FM], fb0[FN], fa1[FM], fb1[FN];
        TZL_READ_FRAGS(fa0, fb0, 0)
        __builtin_amdgcn_s_waitcnt(TK_LGKMCNT0_IMM);

        int c = 0;
        for (; c + STAGES < kchunks; c += 2) {
            TZL_ITERATION(fa0, fb0, fa1, fb1, c, L * (STAGES - 2), true)
            TZL_ITERATION(fa1, fb1, fa0, fb0, c + 1, L * (STAGES - 2), true)
        }
        // the last four chunks: nothing left to fetch, fewer loads in flight
        TZL_ITERATION(fa0, fb0, fa1, fb1, c, L * 2, false)
        TZL_ITERATION(fa1, fb1, fa0, fb0, c + 1, L * 1, false)
        TZL_ITERATION(fa0, fb0, fa1, fb1, c + 2, 0, false)
        _Pragma("unroll") for (int n = 0; n < FM * FN; ++n) { TZL_MFMA_AT(fa1, fb1, n) }
        __builtin_amdgcn_s_barrier();   // every wave is done reading before the next tile refills the ring
        asm volatile("" ::: "memory");

        // lane holds C[row0 + 16 i + lane % 16][col0 + 16 j + 4 (lane / 16) .. + 3]
        float *c_lane = C + (size_t)(mi * TM + wr * (FM * 16) + (lane & 15)) * N + mj * TN + wc * (FN * 16) +
                        (lane >> 4) * 4;
#pragma unroll
        for (int ri = 0; ri < FM / 4; ++ri)
#pragma unroll
            for (int rj = 0; rj < FN / 4; ++rj) {
                const int pos = (ref_r0 + ri) * ref_cols + ref_c0 + rj;
                if (pos < tile_start || pos >= tile_end) continue;   // uniform over the wave
#pragma unroll
                for (int i = 4 * ri; i < 4 * ri + 4; ++i)
#pragma unroll
                    for (int j = 4 * rj; j < 4 * rj + 4; ++j) {
                        float4_t v = acc[i][j] * TZ_ALPHA;
                        float4_t *c_at = reinterpret_cast<float4_t *>(c_lane + (size_t)(i * 16) * N + j * 16);
                        if constexpr (STREAM_C) __builtin_nontemporal_store(v, c_at);
                        else *c_at = v;
                    }
            }
        // stores and LDS-direct loads share the vmcnt counter: drain it so that the counts of
        // the next tile's ring are exact
        __builtin_amdgcn_s_waitcnt(TK_VMCNT_IMM(0));
#undef TZL_ISSUE_CHUNK
#undef TZL_READ_FRAGS
#undef TZL_MFMA_AT
#undef TZL_ITERATION
    }
}

}  // namespace tk
