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
// K loop.  The tile's operands travel in pairs of 32-k chunks: one buffer of the LDS ring holds
// 64 k of the tile as rows of 128 bytes, A rows then B rows, (32*FM + 32*FN) * 128 bytes = 64 KiB
// for 256 x 256, and the ring is two buffers.  They are filled by LDS-direct loads
// (global_load_lds_dwordx4: lane l's 16 bytes land at base + 16 l, so one load fills 8 rows),
// each of which takes whole 128-byte lines from 8 matrix rows: the same loads taking 64 bytes
// from 16 rows each move 55 GB/s into a CU, these 86 (a stand-alone load-shape measurement).
// An iteration multiplies one chunk, whose fragments the wave already holds in registers, and
// meanwhile reads the fragments of the next chunk.  In the first iteration of a pair those come
// from the same buffer, which was published an iteration ago: no wait, no barrier.  In the second
// the wave (i) waits until its own loads of the next pair have landed (vmcnt) and meets the other
// waves at the barrier -- after which the next pair is whole and nobody reads this pair's buffer
// any more -- (ii) reads the first fragments of the next pair and (iii) starts the loads of the
// pair after that into the buffer this pair leaves.  So a pair is fetched while a pair is
// multiplied, there is one barrier per 128 MFMAs of a wave, and it sits behind the first MFMAs of
// its iteration.  The LDS reads follow every third MFMA (the LDS returns 1 KiB to a SIMD in
// about 32 cycles, and the four waves read in step), the loads every third MFMA behind the
// barrier, and every MFMA is fenced with sched_barrier so that the issue order is the source
// order.
//
// The barrier is the hardware one: a counter in LDS with a split arrive / wait (what the
// wave-split fused kernels use) was measured here too and lost 15 % -- its atomics and polls
// queue behind the ring traffic.
//
// LDS layout.  Slot (row, s) of a buffer holds the row's 16-byte k segment s ^ ((row >> 1) & 7):
// the 16 rows a fragment read touches with one k segment then cover all 64 banks once, and the
// hardware counts no bank conflict.  The swizzle is applied on the global side of the
// LDS-direct load (a lane fetches the segment that belongs in the slot it will write) and
// undone by the fragment read.
#pragma once
#include "tzgemm_role.h"

#define TZL_LOOP_LOAD(...) tz_load_to_lds(__VA_ARGS__)
#define TZL_LOOP_READ(dst_, src_) dst_ = src_

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

// Sync: the barrier among the role's four waves -- WorkgroupSync (the hardware barrier) when the
// role owns every wave of its workgroup, RoleHandoverSync inside a wave-split fused kernel.
// stream_c: C leaves with nontemporal stores.  Pays when C is larger than the caches can hold
// until the memory has taken it (256 MiB at 8192 x 8192: plain stores push the operand panels out
// of the L2s); below that plain stores are the faster ones -- the L2s and the memory-side cache
// take the tile at once and write it back while the next kernel already runs (4096 x 4096 x 1024:
// 37 instead of 43 us).
template <int FM, int FN, class Sync>
__device__ __forceinline__ void tzgemm_role_large(const _Float16 *__restrict__ A, const _Float16 *__restrict__ B,
                                                  float *__restrict__ C, int M, int N, int K, int role_block,
                                                  int role_blocks, int tile_start, int tile_end, int tid,
                                                  char *lds, bool stream_c, Sync &sync)
{
    typedef __attribute__((address_space(3))) void *lptr_t;
    constexpr int TM = 32 * FM, TN = 32 * FN;      // macro tile
    constexpr int BK = 32;                         // k of one MFMA step (a chunk)
    constexpr int ROWB = 4 * BK;                   // 128-byte tile rows: a pair of chunks
    constexpr int A_BYTES = TM * ROWB;
    constexpr int PAIR_BYTES = (TM + TN) * ROWB;   // one buffer of the ring: 64 KiB for 256 x 256
    constexpr int LA = TM / 8 / 4;                 // LDS-direct loads per wave and pair: A ...
    constexpr int LB = TN / 8 / 4;                 // ... and B (one load = 8 rows of 128 bytes)
    constexpr int L = LA + LB;
    constexpr int FIRST = 8;                       // MFMAs of an iteration in front of the barrier
    // one LDS read per READ_GAP MFMAs: 3 where the iteration is long enough, else as many as fit
    constexpr int READ_GAP = (FM * FN - FIRST) / (FM + FN) >= 3 ? 3 : (FM * FN - FIRST) / (FM + FN);
    constexpr int LOAD_GAP = (FM * FN - FIRST) / L;
    static_assert(FM % 4 == 0 && FN % 4 == 0, "a wave tile is whole reference tiles");
    static_assert(LA <= 8 && LB <= 8, "eight row blocks of 8 per wave and operand at most");
    static_assert(L < 64, "vmcnt is a 6-bit counter");
    static_assert(READ_GAP >= 1 && (FM + FN) * READ_GAP <= FM * FN - FIRST && LOAD_GAP >= 1,
                  "an iteration slots its LDS reads and loads between the MFMAs behind the barrier");
    static_assert(2 * PAIR_BYTES <= TZ_LDS_BYTES, "the ring is two buffers");

    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wr = wave >> 1;
    const int wc = wave & 1;
    const int ref_cols = N / TZ_REF_TILE;
    const int tile_rows = M / TM;
    const int tile_cols = N / TN;
    const int n_tiles = tile_rows * tile_cols;
    const int npairs = K / (2 * BK);               // K is a multiple of 128: an even number of pairs

    // LDS-direct load map: load j of an operand fills rows 8 (4 j + wave) .. + 7 of its area of the
    // buffer; lane l lands in row + l / 8, slot l % 8 and therefore fetches the 16-byte k segment
    // (l % 8) ^ ((row >> 1) & 7), and (row >> 1) & 7 = l / 16 + 4 (wave % 2) whatever j is.  Per load a
    // 32-bit lane offset below a wave-uniform pointer to the pair of chunks: a load is "scalar base
    // + vector offset" and costs no address arithmetic of its own.
    const unsigned src_lane =
        (unsigned)((lane >> 3) * K + (((lane & 7) ^ ((lane >> 4) | ((wave & 1) << 2))) * 8)) * 2u;
    unsigned src_blk[LA > LB ? LA : LB];
#pragma unroll
    for (int j = 0; j < (LA > LB ? LA : LB); ++j) src_blk[j] = src_lane + (unsigned)((4 * j + wave) * 8) * (unsigned)K * 2u;
    const unsigned lds_dst = (unsigned)(size_t)(lptr_t)lds + wave * 1024;   // + buffer, operand, 4096 j
    // fragment reads: row r = lane % 16 of a 16-row group, k segment lane / 16 of chunk h of the
    // pair, found in slot (4 h + lane / 16) ^ ((r >> 1) & 7)
    const int frag_row = (lane & 15) * ROWB;
    const int frag_h0 = frag_row + (((lane >> 4) ^ ((lane & 15) >> 1)) * 16);
    const int frag_h1 = frag_row + (((4 + (lane >> 4)) ^ ((lane & 15) >> 1)) * 16);
    const int off_a = wr * (FM * 16) * ROWB;
    const int off_b = A_BYTES + wc * (FN * 16) * ROWB;

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

// all loads of the pair of chunks a_ptr_ / b_ptr_ point at, into buffer buf_
#define TZL_ISSUE_PAIR(a_ptr_, b_ptr_, buf_)                                                      \
    {                                                                                             \
        _Pragma("unroll") for (int q = 0; q < LA; ++q)                                            \
            tz_load_to_lds(a_ptr_, src_blk[q], lds_dst + (buf_) * PAIR_BYTES + q * 4096);         \
        _Pragma("unroll") for (int q = 0; q < LB; ++q)                                            \
            tz_load_to_lds(b_ptr_, src_blk[q], lds_dst + (buf_) * PAIR_BYTES + A_BYTES + q * 4096); \
    }
// fragment i of A / j of B of chunk h_ (its lane offset frag_) in buffer buf_
#define TZL_FRAG_A(buf_, frag_, i_) \
    *reinterpret_cast<const half8_t *>(lds + (buf_) * PAIR_BYTES + off_a + (frag_) + (i_) * 16 * ROWB)
#define TZL_FRAG_B(buf_, frag_, j_) \
    *reinterpret_cast<const half8_t *>(lds + (buf_) * PAIR_BYTES + off_b + (frag_) + (j_) * 16 * ROWB)
// MFMA n of an iteration updates accumulator tile (n / FN, n % FN)
#define TZL_MFMA_AT(fa_, fb_, n_)                                                                 \
    acc[(n_) / FN][(n_) % FN] = __builtin_amdgcn_mfma_f32_16x16x32_f16(                           \
        fb_[(n_) % FN], fa_[(n_) / FN], acc[(n_) / FN][(n_) % FN], 0, 0, 0);
// First iteration of a pair: multiply its first chunk (fragments fc_) and read the fragments of
// its second chunk (into fn_) from the same buffer -- landed and published an iteration ago, so
// no wait and no barrier.
#define TZL_ITERATION_FIRST(fc_a_, fc_b_, fn_a_, fn_b_, buf_)                                     \
    {                                                                                             \
        _Pragma("unroll") for (int n = 0; n < FM * FN; ++n)                                       \
        {                                                                                         \
            TZL_MFMA_AT(fc_a_, fc_b_, n)                                                          \
            if (n % READ_GAP == 0 && n / READ_GAP < FM)                                           \
                TZL_LOOP_READ(fn_a_[n / READ_GAP], TZL_FRAG_A(buf_, frag_h1, n / READ_GAP));      \
            else if (n % READ_GAP == 0 && n / READ_GAP < FM + FN)                                 \
                TZL_LOOP_READ(fn_b_[n / READ_GAP - FM], TZL_FRAG_B(buf_, frag_h1, n / READ_GAP - FM)); \
            __builtin_amdgcn_sched_barrier(0);                                                    \
        }                                                                                         \
        __builtin_amdgcn_s_waitcnt(TK_LGKMCNT0_IMM);                                              \
    }
// Second iteration of a pair: multiply its second chunk; behind the first MFMAs wait for this
// wave's loads of the next pair and meet the other waves -- from then on the next pair is whole
// in buffer nbuf_ and nobody reads this pair's buffer buf_ any more -- then read the first
// fragments of the next pair and, if do_issue_, start the loads of the pair a_next / b_next
// point at into buf_.
#define TZL_ITERATION_SECOND(fc_a_, fc_b_, fn_a_, fn_b_, buf_, nbuf_, do_issue_)                  \
    {                                                                                             \
        _Pragma("unroll") for (int n = 0; n < FIRST; ++n)                                         \
        {                                                                                         \
            TZL_MFMA_AT(fc_a_, fc_b_, n)                                                          \
            __builtin_amdgcn_sched_barrier(0);                                                    \
        }                                                                                         \
        __builtin_amdgcn_s_waitcnt(TK_VMCNT_IMM(0));                                              \
        sync.wait();                                                                              \
        __builtin_amdgcn_sched_barrier(0);                                                        \
        _Pragma("unroll") for (int n = FIRST; n < FM * FN; ++n)                                   \
        {                                                                                         \
            TZL_MFMA_AT(fc_a_, fc_b_, n)                                                          \
            const int r_ = n - FIRST;                                                             \
            if (r_ % READ_GAP == 0 && r_ / READ_GAP < FM)                                         \
                TZL_LOOP_READ(fn_a_[r_ / READ_GAP], TZL_FRAG_A(nbuf_, frag_h0, r_ / READ_GAP));   \
            else if (r_ % READ_GAP == 0 && r_ / READ_GAP < FM + FN)                               \
                TZL_LOOP_READ(fn_b_[r_ / READ_GAP - FM], TZL_FRAG_B(nbuf_, frag_h0, r_ / READ_GAP - FM)); \
            if (do_issue_ && r_ % LOAD_GAP == LOAD_GAP - 1 && r_ / LOAD_GAP < L) {                \
                const int q_ = r_ / LOAD_GAP;                                                     \
                if (q_ < LA)                                                                      \
                    TZL_LOOP_LOAD(a_next, src_blk[q_], lds_dst + (buf_) * PAIR_BYTES + q_ * 4096); \
                else                                                                              \
                    TZL_LOOP_LOAD(b_next, src_blk[q_ - LA],                                       \
                                  lds_dst + (buf_) * PAIR_BYTES + A_BYTES + (q_ - LA) * 4096);    \
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

        // fill both buffers (npairs >= 2 always), publish pair 0, fetch its first fragments
        const char *a_next = a_tile, *b_next = b_tile;   // pair the next loads fetch
        for (int b = 0; b < 2; ++b) {
            TZL_ISSUE_PAIR(a_next, b_next, b)
            a_next += ROWB;
            b_next += ROWB;
        }
        __builtin_amdgcn_s_waitcnt(TK_VMCNT_IMM(L));
        sync.wait();
        half8_t fa0[FM], fb0[FN], fa1[FM], fb1[FN];
#pragma unroll
        for (int i = 0; i < FM; ++i) fa0[i] = TZL_FRAG_A(0, frag_h0, i);
#pragma unroll
        for (int j = 0; j < FN; ++j) fb0[j] = TZL_FRAG_B(0, frag_h0, j);
        __builtin_amdgcn_s_waitcnt(TK_LGKMCNT0_IMM);

        // pairs p, p + 1 live in buffers 0, 1; while they are multiplied pairs p + 2, p + 3 are fetched
        for (int p = 0; p + 2 < npairs; p += 2) {
            TZL_ITERATION_FIRST(fa0, fb0, fa1, fb1, 0)
            TZL_ITERATION_SECOND(fa1, fb1, fa0, fb0, 0, 1, true)
            TZL_ITERATION_FIRST(fa0, fb0, fa1, fb1, 1)
            TZL_ITERATION_SECOND(fa1, fb1, fa0, fb0, 1, 0, true)
        }
        // the last two pairs: nothing left to fetch
        TZL_ITERATION_FIRST(fa0, fb0, fa1, fb1, 0)
        TZL_ITERATION_SECOND(fa1, fb1, fa0, fb0, 0, 1, false)
        TZL_ITERATION_FIRST(fa0, fb0, fa1, fb1, 1)
        _Pragma("unroll") for (int n = 0; n < FM * FN; ++n) { TZL_MFMA_AT(fa1, fb1, n) }
        sync.wait();   // every wave is done reading before the next tile refills the ring

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
                        if (stream_c) __builtin_nontemporal_store(v, c_at);   // uniform
                        else *c_at = v;
                    }
            }
        // The stores stay in flight while the next tile starts: they share the vmcnt counter with
        // the LDS-direct loads, but loads complete in their own order, so "at most L operations
        // outstanding" in the next tile's prologue still means that its first pair has landed.
#undef TZL_ISSUE_PAIR
#undef TZL_FRAG_A
#undef TZL_FRAG_B
#undef TZL_MFMA_AT
#undef TZL_ITERATION_FIRST
#undef TZL_ITERATION_SECOND
    }
    sync.finish();
}

// ---------------------------------------------------------------------------------------
// The large-tile form for a wave-split fused kernel of 512 threads.  Two waves share a SIMD there
// (one of the GEMM, one of the other role), so a lane has 256 registers and the tile is
// 256 x 128: a wave tile of 128 x 64 = 8 x 4 accumulator tiles, 128 registers.  Same ring, same
// loads, same LDS layout and the same bits as tzgemm_role_large (every element still sees its
// chunks of 32 k in ascending order).  What differs is how the fragments are held: two register
// sets of 8 + 4 fragments (96 registers) do not fit beside the accumulators, so there is ONE
// set, and the 32 MFMAs of a chunk run in an order that lets every fragment be replaced as soon
// as it is dead.  The order is two blocks of 4 rows of accumulator tiles, column by column
// within a block:  MFMA n multiplies A fragment i = 4 (n / 16) + n % 4 with B fragment
// j = n % 16 / 4.  Then
//    A0..A3 are dead after MFMAs 12..15,  B0, B1, B2 after 19, 23, 27,
//    A4..A7 after 28..31,                 B3 after 31,
// and the next chunk needs A0..A3 and B0 from its MFMA 0 on, B1 from 4, B2 from 8, B3 from 12
// and A4..A7 from 16.  So an iteration reads the next chunk's A0..A3, B0, B1, B2 behind its
// own MFMAs 12, 14, 16, 18, 20, 23, 27 -- each at least 12 MFMAs before its first use -- and its
// OWN B3, A4..A7 behind its MFMAs 0, 2, 4, 6, 7.  In a pair's second iteration the own-chunk
// reads lie in front of the barrier (they read the buffer that is about to be refilled) and the
// next-chunk reads and the 12 LDS-direct loads of the pair after next behind it, one memory
// instruction per MFMA at most.
// Against the 128 x 128 form of the fused kernels a workgroup moves 3/4 of the operand bytes per
// flop through the CU's vector-memory path, and a 4096 x 4096 GEMM has its operands fetched 3
// times over the 8 XCDs instead of 4.5 times.
template <class Sync>
__device__ __forceinline__ void tzgemm_role_large_rot(const _Float16 *__restrict__ A, const _Float16 *__restrict__ B,
                                                      float *__restrict__ C, int M, int N, int K, int role_block,
                                                      int role_blocks, int tile_start, int tile_end, int tid,
                                                      char *lds, bool stream_c, Sync &sync)
{
    typedef __attribute__((address_space(3))) void *lptr_t;
    constexpr int FM = 8, FN = 4;
    constexpr int TM = 32 * FM, TN = 32 * FN;      // 256 x 128
    constexpr int BK = 32;
    constexpr int ROWB = 4 * BK;
    constexpr int A_BYTES = TM * ROWB;
    constexpr int B_BYTES = TN * ROWB;
    constexpr int PAIR_BYTES = A_BYTES + B_BYTES;  // 48 KiB a buffer
    // The ring in LDS: A of buffer 0, A of buffer 1, B of buffer 0, B of buffer 1.  With the two
    // buffers of an operand next to each other every fragment read is "one of four lane addresses
    // (operand, half) + an immediate below 64 KiB", and four address registers serve the loop.
    constexpr int B_BASE = 2 * A_BYTES;
    constexpr int LA = TM / 8 / 4;                 // 8 loads of A ...
    constexpr int LB = TN / 8 / 4;                 // ... and 4 of B per wave and pair
    constexpr int L = LA + LB;
    constexpr int NM = FM * FN;                    // 32 MFMAs an iteration
    constexpr int FIRST = 8;                       // MFMAs of a pair's second iteration in front of the barrier
    static_assert(2 * PAIR_BYTES <= TZ_LDS_BYTES, "the ring is two buffers");

    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wr = wave >> 1;
    const int wc = wave & 1;
    const int ref_cols = N / TZ_REF_TILE;
    const int tile_rows = M / TM;
    const int tile_cols = N / TN;
    const int n_tiles = tile_rows * tile_cols;
    const int npairs = K / (2 * BK);

    // LDS-direct load q of an operand fills rows 8 (4 q + wave) .. + 7 of its area (tzgemm_role_large);
    // here the row block 32 q is part of the wave-uniform base (scalar arithmetic) and one lane offset
    // serves every load
    const unsigned src_lane = (unsigned)(((lane >> 3) + 8 * wave) * K + (((lane & 7) ^ ((lane >> 4) | ((wave & 1) << 2))) * 8)) * 2u;
    const size_t block_stride = (size_t)64 * (size_t)K;   // bytes between the rows of loads q and q + 1
    const unsigned lds_dst = (unsigned)(size_t)(lptr_t)lds + wave * 1024;
    const int frag_row = (lane & 15) * ROWB;
    const int frag_h0 = frag_row + (((lane >> 4) ^ ((lane & 15) >> 1)) * 16);
    const int frag_h1 = frag_row + (((4 + (lane >> 4)) ^ ((lane & 15) >> 1)) * 16);
    const int off_a = wr * (FM * 16) * ROWB;
    const int off_b = B_BASE + wc * (FN * 16) * ROWB;

    for (int t = role_block; t < n_tiles; t += role_blocks) {
        int mi, mj;
        tz_large_tile_of(t, tile_rows, tile_cols, mi, mj);
        const int ref_r0 = mi * (TM / TZ_REF_TILE) + wr * (FM / 4);
        const int ref_c0 = mj * (TN / TZ_REF_TILE) + wc * (FN / 4);
        {
            const int r_first = mi * (TM / TZ_REF_TILE), c_first = mj * (TN / TZ_REF_TILE);
            bool any = false;
            for (int r = 0; r < TM / TZ_REF_TILE; ++r) {
                const int p0 = (r_first + r) * ref_cols + c_first;
                any |= p0 < tile_end && p0 + TN / TZ_REF_TILE > tile_start;
            }
            if (!any) continue;   // uniform over the workgroup
        }
        const char *a_tile = reinterpret_cast<const char *>(A + (size_t)(mi * TM) * K);
        const char *b_tile = reinterpret_cast<const char *>(B + (size_t)(mj * TN) * K);

#define TZR_LOAD(q_, buf_)                                                                        \
    {                                                                                             \
        if ((q_) < LA)                                                                            \
            tz_load_to_lds(a_next + (size_t)(q_) * block_stride, src_lane, lds_dst + (buf_) * A_BYTES + (q_) * 4096); \
        else                                                                                      \
            tz_load_to_lds(b_next + (size_t)((q_) - LA) * block_stride, src_lane,                 \
                           lds_dst + B_BASE + (buf_) * B_BYTES + ((q_) - LA) * 4096);             \
    }
#define TZR_FRAG_A(buf_, frag_, i_) \
    *reinterpret_cast<const half8_t *>(lds + off_a + (frag_) + (buf_) * A_BYTES + (i_) * 16 * ROWB)
#define TZR_FRAG_B(buf_, frag_, j_) \
    *reinterpret_cast<const half8_t *>(lds + off_b + (frag_) + (buf_) * B_BYTES + (j_) * 16 * ROWB)
// MFMA n of an iteration: accumulator tile (4 (n / 16) + n % 4, n % 16 / 4)
#define TZR_MFMA(n_)                                                                              \
    {                                                                                             \
        constexpr int i_ = 4 * ((n_) / 16) + (n_) % 4, j_ = ((n_) % 16) / 4;                      \
        acc[i_][j_] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb[j_], fa[i_], acc[i_][j_], 0, 0, 0); \
    }
// reads of the chunk that is being multiplied (half frag_ of buffer buf_): B3 and A4..A7, behind MFMA n_
#define TZR_OWN_READS(n_, buf_, frag_)                                                            \
    {                                                                                             \
        if ((n_) == 0) fb[3] = TZR_FRAG_B(buf_, frag_, 3);                                        \
        if ((n_) == 2) fa[4] = TZR_FRAG_A(buf_, frag_, 4);                                        \
        if ((n_) == 4) fa[5] = TZR_FRAG_A(buf_, frag_, 5);                                        \
        if ((n_) == 6) fa[6] = TZR_FRAG_A(buf_, frag_, 6);                                        \
        if ((n_) == 7) fa[7] = TZR_FRAG_A(buf_, frag_, 7);                                        \
    }
// reads of the next chunk (half frag_ of buffer buf_): A0..A3, B0, B1, B2, behind MFMA n_
#define TZR_NEXT_READS(n_, buf_, frag_)                                                           \
    {                                                                                             \
        if ((n_) == 12) fa[0] = TZR_FRAG_A(buf_, frag_, 0);                                       \
        if ((n_) == 14) fa[1] = TZR_FRAG_A(buf_, frag_, 1);                                       \
        if ((n_) == 16) fa[2] = TZR_FRAG_A(buf_, frag_, 2);                                       \
        if ((n_) == 18) fa[3] = TZR_FRAG_A(buf_, frag_, 3);                                       \
        if ((n_) == 20) fb[0] = TZR_FRAG_B(buf_, frag_, 0);                                       \
        if ((n_) == 23) fb[1] = TZR_FRAG_B(buf_, frag_, 1);                                       \
        if ((n_) == 27) fb[2] = TZR_FRAG_B(buf_, frag_, 2);                                       \
    }
// A pair's first iteration: its second chunk lies in the same buffer, published an iteration ago --
// no wait and no barrier.
#define TZR_ITERATION_FIRST(buf_)                                                                 \
    {                                                                                             \
        _Pragma("unroll") for (int n = 0; n < NM; ++n)                                            \
        {                                                                                         \
            TZR_MFMA_AT(n)                                                                        \
            TZR_OWN_READS(n, buf_, frag_h0)                                                       \
            TZR_NEXT_READS(n, buf_, frag_h1)                                                      \
            __builtin_amdgcn_sched_barrier(0);                                                    \
        }                                                                                         \
    }
// A pair's second iteration: behind the first MFMAs wait for this wave's loads of the next pair
// and for its own LDS reads, and meet the other waves -- the next pair is then whole in nbuf_ and
// nobody reads buf_ any more; read the next pair's first fragments and, if do_issue_, start the
// loads of the pair after that into buf_.
#define TZR_ITERATION_SECOND(buf_, nbuf_, do_issue_)                                              \
    {                                                                                             \
        _Pragma("unroll") for (int n = 0; n < FIRST; ++n)                                         \
        {                                                                                         \
            TZR_MFMA_AT(n)                                                                        \
            TZR_OWN_READS(n, buf_, frag_h1)                                                       \
            __builtin_amdgcn_sched_barrier(0);                                                    \
        }                                                                                         \
        __builtin_amdgcn_s_waitcnt(TK_VMCNT_IMM(0));                                              \
        sync.sync();                                                                              \
        __builtin_amdgcn_sched_barrier(0);                                                        \
        _Pragma("unroll") for (int n = FIRST; n < NM; ++n)                                        \
        {                                                                                         \
            TZR_MFMA_AT(n)                                                                        \
            TZR_NEXT_READS(n, nbuf_, frag_h0)                                                     \
            if (do_issue_) {                                                                      \
                constexpr int slot_[L] = {9, 11, 13, 15, 17, 19, 21, 22, 25, 26, 29, 31};         \
                _Pragma("unroll") for (int q = 0; q < L; ++q)                                     \
                    if (n == slot_[q]) TZR_LOAD(q, buf_)                                          \
            }                                                                                     \
            __builtin_amdgcn_sched_barrier(0);                                                    \
        }                                                                                         \
        if (do_issue_) {                                                                          \
            a_next += ROWB;                                                                       \
            b_next += ROWB;                                                                       \
        }                                                                                         \
    }
// (the loop variable of an unrolled loop is a constant the MFMA's tile indices are computed from)
#define TZR_MFMA_AT(n_)                                                                           \
    {                                                                                             \
        const int i_ = 4 * ((n_) / 16) + (n_) % 4, j_ = ((n_) % 16) / 4;                          \
        acc[i_][j_] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb[j_], fa[i_], acc[i_][j_], 0, 0, 0); \
    }

        float4_t acc[FM][FN];
#pragma unroll
        for (int i = 0; i < FM; ++i)
#pragma unroll
            for (int j = 0; j < FN; ++j) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};

        // fill both buffers (npairs >= 2 always), publish pair 0, fetch what its first chunk does
        // not read itself
        const char *a_next = a_tile, *b_next = b_tile;
        for (int b = 0; b < 2; ++b) {
            _Pragma("unroll") for (int q = 0; q < L; ++q) TZR_LOAD(q, b)
            a_next += ROWB;
            b_next += ROWB;
        }
        __builtin_amdgcn_s_waitcnt(TK_VMCNT_IMM(L));
        sync.sync();
        half8_t fa[FM], fb[FN];
#pragma unroll
        for (int i = 0; i < 4; ++i) fa[i] = TZR_FRAG_A(0, frag_h0, i);
#pragma unroll
        for (int j = 0; j < 3; ++j) fb[j] = TZR_FRAG_B(0, frag_h0, j);

        for (int p = 0; p + 2 < npairs; p += 2) {
            TZR_ITERATION_FIRST(0)
            TZR_ITERATION_SECOND(0, 1, true)
            TZR_ITERATION_FIRST(1)
            TZR_ITERATION_SECOND(1, 0, true)
        }
        // the last two pairs: nothing left to fetch, and behind the last chunk nothing left to read
        TZR_ITERATION_FIRST(0)
        TZR_ITERATION_SECOND(0, 1, false)
        TZR_ITERATION_FIRST(1)
        _Pragma("unroll") for (int n = 0; n < NM; ++n)
        {
            TZR_MFMA_AT(n)
            TZR_OWN_READS(n, 1, frag_h1)
            __builtin_amdgcn_sched_barrier(0);
        }
        sync.sync();   // every wave is done reading before the next tile refills the ring

        // (the lane's share of the address is formed here, from the lane number read afresh: nothing of
        // it is kept in registers across the K loop)
        int lane_here;
        asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(lane_here));
        float *c_lane = C + (size_t)(mi * TM + wr * (FM * 16) + (lane_here & 15)) * N + mj * TN + wc * (FN * 16) +
                        (lane_here >> 4) * 4;
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
                        if (stream_c) __builtin_nontemporal_store(v, c_at);   // uniform
                        else *c_at = v;
                        // one tile at a time: scaled, stored, its registers free again (left to itself the
                        // compiler scales all 32 tiles first, and 128 more registers do not exist here)
                        __builtin_amdgcn_sched_barrier(0);
                    }
            }
        // (the stores stay in flight while the next tile starts, as in tzgemm_role_large)
#undef TZR_LOAD
#undef TZR_FRAG_A
#undef TZR_FRAG_B
#undef TZR_MFMA
#undef TZR_MFMA_AT
#undef TZR_OWN_READS
#undef TZR_NEXT_READS
#undef TZR_ITERATION_FIRST
#undef TZR_ITERATION_SECOND
    }
    sync.finish();
}

}  // namespace tk
