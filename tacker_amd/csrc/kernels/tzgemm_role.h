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
// gfx950 design.  A 256-thread role (4 wave64) owns a 128x128 macro tile = 2x2
// reference tiles; wave (wr,wc) computes reference tile (2*mi+wr, 2*mj+wc) with
// 4x4 v_mfma_f32_16x16x32_f16 accumulators.  A and B both have K contiguous,
// which is the operand layout MFMA wants (lane l supplies 8 consecutive k of row
// l%16), so tiles go to LDS as they are.
//
// Three things keep the MFMA pipe fed with one GEMM wave per SIMD:
//  * global latency -- the K loop is a ring of STAGES LDS stages (64 k each,
//    32 KiB) filled by global_load_lds_dwordx4: the load writes LDS directly,
//    costs no VGPRs, and almost STAGES-1 chunks are in flight while one is
//    multiplied.  A wave knows its loads of a chunk have landed from the vmcnt
//    counter (s_waitcnt vmcnt(8*(STAGES-2))), then one role barrier publishes
//    the chunk.
//  * LDS latency -- fragments are double-buffered in registers: the 8
//    ds_read_b128 of the next k-step are issued between the first MFMAs of the
//    current one, so the wave never sits idle between its LDS reads and its MFMAs.
//  * issue slots -- a wave issues in order and blocks at a load while the CU's
//    vector-memory queue is full, so the 8 loads of a chunk go out one at a time
//    behind individual MFMAs, 4 in each k-step, with scalar address arithmetic only.
// An LDS-direct load puts lane l's 16 bytes at base + 16*l, so tile rows are dense
// (128 B); bank conflicts are avoided by a swizzle applied on the global side:
// LDS slot (row, s) holds the row's 16-byte segment s ^ ((row >> 1) & 7), and the
// fragment read undoes it.
//
// The MFMA is issued with the operands swapped (B fragment first) so each lane
// ends up with 4 consecutive columns of one row of C and stores 16 bytes at once.
// A wave stores its tile only if the tile's position is inside the range; macro
// tiles with no position in range are skipped by the whole workgroup.
//
// Shapes with few tiles and a long reduction take a second form (tzgemm_role_ksplit,
// below): one reference tile per workgroup, K cut over its 4 waves.
#pragma once
#include "role_common.h"
#include "../header/tzgemm_header.h"

// Output buffer -> workspace, filled by the host when it binds a workspace to a C
// (tzgemmWorkspaceFor); see tz_ws_entry.
__device__ tz_ws_entry tz_ws_table[TZ_WS_TABLE_SLOTS];

namespace tk {

// The workspace bound to a key of the table (tz_ws_key_*), nullptr if there is none.  The key comes
// from a kernel argument, so the probes are scalar loads; the host never lets a key sit more than
// TZ_WS_TABLE_MAX_PROBES slots from its hash, and a binding it takes out leaves a tombstone that
// the probe walks past.
__device__ __forceinline__ unsigned *tz_find_workspace(unsigned long long key)
{
    unsigned slot = tz_ws_hash(key);
    for (int probe = 0; probe < TZ_WS_TABLE_MAX_PROBES; ++probe) {
        const unsigned long long c = tz_ws_table[slot].c;
        if (c == key) return reinterpret_cast<unsigned *>((size_t)tz_ws_table[slot].workspace);
        if (c == 0ull) return nullptr;
        slot = (slot + 1) & (TZ_WS_TABLE_SLOTS - 1);
    }
    return nullptr;
}
// ... for a GEMM of this shape: only the shapes whose reduction is shared by workgroups look.
__device__ __forceinline__ unsigned *tz_workspace_of(const float *C, int M, int N, int K)
{
    return tz_ksplit_parts(M, N, K) > 1 ? tz_find_workspace(tz_ws_key_tzgemm(C)) : nullptr;
}

// Persistent-loop index -> macro tile (row, column).  With role_blocks a multiple
// of 8, loop index t runs on XCD t % 8.  Each XCD takes a contiguous run of the
// tile sequence, and the sequence walks the tile grid in bands of 4 tile rows,
// column by column, so the ~32 tiles an XCD works on at the same time form a
// compact 4 x 8 block: they share 4 A row panels and 8 B column panels inside
// that XCD's L2 instead of streaming a whole operand through it.
__device__ __forceinline__ void tz_macro_tile_of(int t, int macro_rows, int macro_cols, int &mi, int &mj)
{
    const int n_macro = macro_rows * macro_cols;
    int seq = t;
    if (n_macro % TK_XCD_NUM == 0) seq = (t % TK_XCD_NUM) * (n_macro / TK_XCD_NUM) + t / TK_XCD_NUM;
    const int band = (macro_rows % 4 == 0) ? 4 : ((macro_rows % 2 == 0) ? 2 : 1);
    const int per_band = band * macro_cols;
    const int in_band = seq % per_band;
    mi = (seq / per_band) * band + in_band % band;
    mj = in_band / band;
}

// s_waitcnt immediate that waits for vmcnt <= n and leaves expcnt / lgkmcnt alone
#define TK_VMCNT_IMM(n) (((n) & 15) | (((n) >> 4) << 14) | 0x0F70)
// s_waitcnt immediate that waits for lgkmcnt == 0 (LDS reads landed) and nothing else
#define TK_LGKMCNT0_IMM 0xC07F

// One LDS-direct load of 16 bytes per lane: global address = scalar base + 32-bit lane
// offset (an addressing mode of the instruction, so no 64-bit vector address is formed and
// no VALU work is spent on it), LDS address = scalar (M0).  Written as asm because the
// builtin only selects the vector-address form.  The compiler does not count these loads
// in vmcnt; the role waits for them with explicit s_waitcnt.
__device__ __forceinline__ void tz_load_to_lds(const char *uniform_base, unsigned lane_offset, unsigned lds_address)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_address), "v"(lane_offset), "s"(uniform_base)
                 : "memory");
}

// the same with the nontemporal hint: for an operand that is read once (the weights of a fully
// connected layer at batch 1)
__device__ __forceinline__ void tz_load_to_lds_once(const char *uniform_base, unsigned lane_offset, unsigned lds_address)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 nt"
                 :
                 : "s"(lds_address), "v"(lane_offset), "s"(uniform_base)
                 : "memory");
}

template <int STAGES, bool STREAM_C, class Sync>
__device__ __forceinline__ void tzgemm_role_tiles(const _Float16 *__restrict__ A,
                                            const _Float16 *__restrict__ B, float *__restrict__ C,
                                            int M, int N, int K, int role_block, int role_blocks,
                                            int tile_start, int tile_end, int tid, char *lds,
                                            Sync &sync)
{
    typedef __attribute__((address_space(3))) void *lptr_t;
    constexpr int BK = TZ_BLOCK_K;
    constexpr int ROWB = BK * 2;                         // dense 128-byte tile rows
    constexpr int OPERAND_BYTES = TZ_MACRO_TILE * ROWB;  // 16 KiB
    constexpr int STAGE_BYTES = TZ_STAGE_BYTES;
    constexpr int LOADS = 4;                             // LDS-direct loads per wave, operand and chunk
    constexpr int LOADS_PER_CHUNK = 2 * LOADS;
    static_assert(STAGES >= 3 && LOADS_PER_CHUNK * (STAGES - 2) < 64, "vmcnt is a 6-bit counter");

    const int lane = tid & 63;
    // wave-uniform by construction: everything derived from it (the LDS address an
    // LDS-direct load goes to, i.e. M0) then stays in scalar registers
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wr = wave >> 1;
    const int wc = wave & 1;
    const int ref_cols = N / TZ_REF_TILE;
    const int macro_cols = N / TZ_MACRO_TILE;
    const int n_macro = (M / TZ_MACRO_TILE) * macro_cols;
    const int kchunks = K / BK;

    // LDS-direct load map.  Load j (0..3) of this wave fills rows (4*wave+j)*8 ..+7 of an
    // operand's stage area; lane l lands in row +l/8, slot l%8, and therefore fetches the
    // row's segment slot ^ ((row>>1)&7).  Rows of consecutive loads are 8 apart, which flips
    // bit 2 of the key: odd loads fetch segment (seg ^ 4).
    const int dma_row = 4 * wave * 8 + (lane >> 3);
    const int dma_seg = (lane & 7) ^ ((dma_row >> 1) & 7);
    // per-lane byte offsets below a wave-uniform row-block address (even / odd loads); kept as
    // 32-bit offsets so a load is "scalar base + vector offset" and holds no 64-bit pointers
    const unsigned src_even = (unsigned)(dma_row * K + dma_seg * 8) * 2u;
    const unsigned src_odd = (unsigned)(dma_row * K + (dma_seg ^ 4) * 8) * 2u;
    const int dst_off = 4 * wave * 1024;                        // + j*1024 per load
    const unsigned lds_base = (unsigned)(size_t)(lptr_t)lds;
    // fragment reads: row r = lane%16 of a 16-row group (its swizzle key (r>>1)&7 is the
    // same in every group), k segment 4*kstep + lane/16 of the 8 in a row
    const int frag_key = ((lane & 15) >> 1) & 7;
    const int frag_seg0 = ((lane >> 4) ^ frag_key) * 16;
    const int frag_seg1 = ((4 + (lane >> 4)) ^ frag_key) * 16;
    const int frag_a = (wr * 64 + (lane & 15)) * ROWB;
    const int frag_b = OPERAND_BYTES + (wc * 64 + (lane & 15)) * ROWB;

    for (int t = role_block; t < n_macro; t += role_blocks) {
        int mi, mj;
        tz_macro_tile_of(t, M / TZ_MACRO_TILE, macro_cols, mi, mj);
        const int pos00 = (2 * mi) * ref_cols + 2 * mj;
        const int pos10 = pos00 + ref_cols;
        const bool in00 = pos00 >= tile_start && pos00 < tile_end;
        const bool in01 = pos00 + 1 >= tile_start && pos00 + 1 < tile_end;
        const bool in10 = pos10 >= tile_start && pos10 < tile_end;
        const bool in11 = pos10 + 1 >= tile_start && pos10 + 1 < tile_end;
        if (!(in00 || in01 || in10 || in11)) continue;   // uniform over the workgroup
        const bool store = wr ? (wc ? in11 : in10) : (wc ? in01 : in00);

        const char *a_tile = reinterpret_cast<const char *>(A + (size_t)(mi * TZ_MACRO_TILE) * K);
        const char *b_tile = reinterpret_cast<const char *>(B + (size_t)(mj * TZ_MACRO_TILE) * K);

// load q (0..7) of a chunk: operand q&1 (A, B), row block j = q>>1
#define TZ_ISSUE_ONE(chunk_, stage_, q_)                                                          \
    {                                                                                             \
        const int j_ = (q_) >> 1;                                                                 \
        const size_t uni_ = ((size_t)(j_ * 8) * K + (size_t)(chunk_) * BK) * 2;                   \
        const unsigned dst_ = lds_base + (stage_) * STAGE_BYTES + dst_off + j_ * 1024 +           \
                              (((q_) & 1) ? OPERAND_BYTES : 0);                                   \
        tz_load_to_lds((((q_) & 1) ? b_tile : a_tile) + uni_, (j_ & 1) ? src_odd : src_even, dst_); \
    }
#define TZ_LOOP_ISSUE_ONE(chunk_, stage_, q_) TZ_ISSUE_ONE(chunk_, stage_, q_)
#define TZ_ISSUE_CHUNK(chunk_, stage_)                                                            \
    _Pragma("unroll") for (int q = 0; q < LOADS_PER_CHUNK; ++q) TZ_ISSUE_ONE(chunk_, stage_, q)
#define TZ_READ_FRAGS(fa_, fb_, stage_, seg_)                                                     \
    _Pragma("unroll") for (int i = 0; i < 4; ++i)                                                 \
    {                                                                                             \
        const char *s_ = lds + (stage_) * STAGE_BYTES + i * 16 * ROWB + (seg_);                   \
        fa_[i] = *reinterpret_cast<const half8_t *>(s_ + frag_a);                                 \
        fb_[i] = *reinterpret_cast<const half8_t *>(s_ + frag_b);                                 \
    }
#define TZ_MFMAS_ROWS(fa_, fb_, i0_, i1_)                                                         \
    _Pragma("unroll") for (int i = i0_; i < i1_; ++i) _Pragma("unroll") for (int j = 0; j < 4; ++j) \
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb_[j], fa_[i], acc[i][j], 0, 0, 0);
#define TZ_MFMAS(fa_, fb_) TZ_MFMAS_ROWS(fa_, fb_, 0, 4)
// Issue order inside one scheduling region: after each MFMA one LDS read (count_ of them),
// then after each MFMA one LDS-direct load (count2_).  An MFMA occupies the matrix pipe for
// 16 cycles but the wave for 4, so the memory instructions slot into its shadow instead
// of queuing up in front of the next MFMA group.
#define TZ_PAIR_MFMA_WITH(mask_, count_)                                                          \
    _Pragma("unroll") for (int q = 0; q < count_; ++q)                                            \
    {                                                                                             \
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                        \
        __builtin_amdgcn_sched_group_barrier(mask_, 1, 0);                                        \
    }
#define TZ_SCHED_DS_READ 0x100
#define TZ_MFMA_AT(fa_, fb_, n_)                                                                  \
    acc[(n_) >> 2][(n_) & 3] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb_[(n_) & 3], fa_[(n_) >> 2], \
                                                                      acc[(n_) >> 2][(n_) & 3], 0, 0, 0);
// First k-step of a chunk multiplied while the chunk barrier completes; the reads of the
// second k-step (into fn_, fbn_) ride in the shadow of the first 8 MFMAs, and loads 4..7 of
// chunk tail_chunk_ (the half of a chunk the previous second k-step did not issue) follow one
// per MFMA.  The 8 loads of a chunk are spread over a whole chunk's worth of MFMAs on purpose:
// the CU's vector-memory unit takes about 10 ns per load, a wave blocks at issue while the
// unit's queue is full, and 32 loads issued right behind the barrier by the four waves at
// once would stall the MFMAs queued behind them.
#define TZ_FIRST_STEP_ACROSS_BARRIER(fa_, fb_, fn_, fbn_, vmcnt_, tail_chunk_, tail_stage_)       \
    TZ_MFMAS_ROWS(fa_, fb_, 0, 2)                                                                 \
    TZ_PAIR_MFMA_WITH(TZ_SCHED_DS_READ, 8)                                                        \
    __builtin_amdgcn_sched_barrier(0);                                                            \
    _Pragma("unroll") for (int q = 0; q < 8; ++q)                                                 \
    {                                                                                             \
        TZ_MFMA_AT(fa_, fb_, 8 + q)                                                               \
        if ((q & 1) == 0 && (tail_chunk_) >= 0) TZ_LOOP_ISSUE_ONE(tail_chunk_, tail_stage_, 4 + q / 2) \
        __builtin_amdgcn_sched_barrier(0);                                                        \
    }                                                                                             \
    __builtin_amdgcn_s_waitcnt(TK_LGKMCNT0_IMM);                                                  \
    __builtin_amdgcn_s_waitcnt(TK_VMCNT_IMM(vmcnt_));                                             \
    sync.wait();
// Second k-step (what is left of it): the 8 reads of the next chunk's first k-step ride
// between its first MFMAs and, if chunk_ >= 0, loads 0..3 of a new chunk follow; its loads
// 4..7 go out with the next first k-step.
#define TZ_SECOND_STEP(fa_, fb_, chunk_, stage_)                                                  \
    TZ_MFMAS_ROWS(fa_, fb_, 0, 2)                                                                 \
    TZ_PAIR_MFMA_WITH(TZ_SCHED_DS_READ, 8)                                                        \
    __builtin_amdgcn_sched_barrier(0);                                                            \
    _Pragma("unroll") for (int q = 0; q < 8; ++q)                                                 \
    {                                                                                             \
        TZ_MFMA_AT(fa_, fb_, 8 + q)                                                               \
        if ((q & 1) == 0 && (chunk_) >= 0) TZ_LOOP_ISSUE_ONE(chunk_, stage_, q / 2)               \
        __builtin_amdgcn_sched_barrier(0);                                                        \
    }

        float4_t acc[4][4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};

        // fill the ring, publish chunk 0, fetch its first k-step.  When the K loop is longer
        // than the ring, the last chunk of the prologue goes out only half (loads 0..3): its
        // other half is the "tail" the first k-step of chunk 0 issues, which puts the loop into
        // its steady rhythm (half a chunk of loads per k-step) without a special first pass.
        const bool ring_runs = kchunks > STAGES;
        const int prologue = ring_runs ? STAGES - 1 : kchunks;
        for (int c = 0; c < prologue; ++c) { TZ_ISSUE_CHUNK(c, c) }
        if (ring_runs) {
            _Pragma("unroll") for (int q = 0; q < 4; ++q) TZ_ISSUE_ONE(STAGES - 1, STAGES - 1, q)
            __builtin_amdgcn_s_waitcnt(TK_VMCNT_IMM(LOADS_PER_CHUNK * (STAGES - 2) + 4));
        } else if (kchunks == STAGES) {
            __builtin_amdgcn_s_waitcnt(TK_VMCNT_IMM(LOADS_PER_CHUNK * (STAGES - 1)));
        } else {
            __builtin_amdgcn_s_waitcnt(TK_VMCNT_IMM(0));
        }
        sync.sync();
        half8_t fa0[4], fb0[4], fa1[4], fb1[4];
        TZ_READ_FRAGS(fa0, fb0, 0, frag_seg0)
        __builtin_amdgcn_s_waitcnt(TK_LGKMCNT0_IMM);

        int stage = 0;   // stage of chunk kc (and of chunk kc+STAGES, refilled once kc is consumed)
        int kc = 0;
        // steady state: chunk kc+STAGES exists.  The first k-step completes chunk kc+STAGES-1
        // (into the stage chunk kc-1 left), after which exactly STAGES-2 chunks of this wave's
        // loads may stay in flight when chunk kc+1 is needed; the second k-step starts chunk
        // kc+STAGES in the stage chunk kc has just left.  Branch-free body.
        for (; kc + STAGES < kchunks; ++kc) {
            const int next_stage = stage + 1 == STAGES ? 0 : stage + 1;
            const int prev_stage = stage == 0 ? STAGES - 1 : stage - 1;
            TZ_READ_FRAGS(fa1, fb1, stage, frag_seg1)     // second k-step of chunk kc, in flight ...
            // ... while the first one is multiplied.  Past the barrier chunk kc+1 is complete
            // in LDS and every wave has read all of chunk kc.
            TZ_FIRST_STEP_ACROSS_BARRIER(fa0, fb0, fa1, fb1, LOADS_PER_CHUNK * (STAGES - 2), kc + STAGES - 1,
                                         prev_stage)
            TZ_READ_FRAGS(fa0, fb0, next_stage, frag_seg0)
            TZ_SECOND_STEP(fa1, fb1, kc + STAGES, stage)
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_waitcnt(TK_LGKMCNT0_IMM);
            stage = next_stage;
        }
        // one more first k-step has a tail to issue: the last chunk's second half
        if (ring_runs) {
            const int next_stage = stage + 1 == STAGES ? 0 : stage + 1;
            const int prev_stage = stage == 0 ? STAGES - 1 : stage - 1;
            TZ_READ_FRAGS(fa1, fb1, stage, frag_seg1)
            TZ_FIRST_STEP_ACROSS_BARRIER(fa0, fb0, fa1, fb1, LOADS_PER_CHUNK * (STAGES - 2), kchunks - 1, prev_stage)
            TZ_READ_FRAGS(fa0, fb0, next_stage, frag_seg0)
            TZ_SECOND_STEP(fa1, fb1, -1, 0)
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_waitcnt(TK_LGKMCNT0_IMM);
            stage = next_stage;
            ++kc;
        }
        // drain: nothing left to issue, fewer loads in flight -- wait for all of them
        for (; kc + 1 < kchunks; ++kc) {
            const int next_stage = stage + 1 == STAGES ? 0 : stage + 1;
            TZ_READ_FRAGS(fa1, fb1, stage, frag_seg1)
            TZ_FIRST_STEP_ACROSS_BARRIER(fa0, fb0, fa1, fb1, 0, -1, 0)
            TZ_READ_FRAGS(fa0, fb0, next_stage, frag_seg0)
            TZ_SECOND_STEP(fa1, fb1, -1, 0)
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_waitcnt(TK_LGKMCNT0_IMM);
            stage = next_stage;
        }
        // last chunk: nothing left to fetch
        TZ_READ_FRAGS(fa1, fb1, stage, frag_seg1)
        TZ_MFMAS(fa0, fb0)
        TZ_MFMAS(fa1, fb1)
        sync.sync();   // all waves are done reading before the next tile refills the ring

        if (store) {
            // lane holds C[row0 + i*16 + lane%16][col0 + j*16 + 4*(lane/16) .. +3]
            float *c_lane = C + (size_t)(mi * TZ_MACRO_TILE + wr * 64 + (lane & 15)) * N +
                            mj * TZ_MACRO_TILE + wc * 64 + (lane >> 4) * 4;
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    float4_t v = acc[i][j] * TZ_ALPHA;
                    // C is written once and not read again by this kernel: as a streaming store it
                    // does not push the operand panels the next tiles need out of the L2 (STREAM_C;
                    // off where the other role of a fused kernel measures better without it)
                    float4_t *c_at = reinterpret_cast<float4_t *>(c_lane + (size_t)(i * 16) * N + j * 16);
                    if constexpr (STREAM_C) __builtin_nontemporal_store(v, c_at);
                    else *c_at = v;
                }
        }
        // stores and LDS-direct loads share the vmcnt counter: drain it so that the
        // counts of the next tile's ring are exact
        __builtin_amdgcn_s_waitcnt(TK_VMCNT_IMM(0));
#undef TZ_ISSUE_CHUNK
#undef TZ_ISSUE_ONE
#undef TZ_LOOP_ISSUE_ONE
#undef TZ_MFMA_AT
#undef TZ_READ_FRAGS
#undef TZ_MFMAS
#undef TZ_MFMAS_ROWS
#undef TZ_PAIR_MFMA_WITH
#undef TZ_SCHED_DS_READ
#undef TZ_FIRST_STEP_ACROSS_BARRIER
#undef TZ_SECOND_STEP
    }
    sync.finish();
}

// ---------------------------------------------------------------------------------------
// K-split form for shapes with few output tiles and a long reduction (the batch-1 layers
// of a network: 8 to 50 macro tiles for 256 CUs, K up to 25088).  The macro-tile form
// would leave most CUs idle and walk K serially on the rest.  Here a workgroup owns ONE
// reference 64x64 tile and its 4 waves each reduce a quarter of K into a private 4x4
// accumulator set, then the four partial tiles are added in LDS in a fixed order
// (((w0 + w1) + w2) + w3), so the result does not depend on timing.  Four times as many
// workgroups, each with a K loop a quarter as long.  The waves share no operands, so each
// has a private two-stage ring (2 x 16 KiB) and the K loop needs no barrier at all.
//
// When even that leaves CUs without work (32 to 128 tiles), the reduction of a tile is
// also cut over tz_ksplit_parts workgroups.  A unit of work is (part, tile); a workgroup
// adds its part of K as above, stores the partial tile to the workspace, and takes a
// ticket from the tile's arrival counter.  The workgroup that draws the last ticket adds
// the partial tiles in part order (((p0 + p1) + p2) ...), scales, stores C and puts the
// counter back to zero: nobody ever waits for another workgroup, and the sum does not
// depend on who came last.
//
// Which form runs, and how many parts, depends on (M, N, K) only -- never on the launch
// geometry -- so a fused launch and the plain kernel always add in the same order.

// Unit of the K-split form a workgroup takes in one round of the persistent loop, -1 for
// none.  count units (at most role_blocks) are handed out; when both are multiples of 8,
// workgroup b runs on XCD b % 8 and each XCD gets a contiguous run of units -- units that
// follow each other share operand panels (same part of K, neighbouring tiles), which then
// meet in that XCD's L2.  Either way the first count workgroups are the ones with a unit.
__device__ __forceinline__ int tz_ksplit_unit_of(int role_block, int role_blocks, int count)
{
    if (role_block >= count) return -1;
    if (role_blocks % TK_XCD_NUM == 0 && count % TK_XCD_NUM == 0)
        return (role_block % TK_XCD_NUM) * (count / TK_XCD_NUM) + role_block / TK_XCD_NUM;
    return role_block;
}

// The same value, but one the compiler has to take as computed here: addresses derived from it
// are formed where they are used instead of being kept in registers across the K loop (the
// sixteen block offsets of a partial tile, hoisted out of the tile loop, do not fit beside the
// accumulators in a fused kernel's 168 registers).
__device__ __forceinline__ int tz_opaque(int v)
{
    asm volatile("" : "+v"(v));
    return v;
}

// Partial tiles travel between workgroups on other XCDs, whose L2s do not see each other's
// lines.  Every access to them is an agent-scope access of its own (it goes through to the
// memory side both XCDs share), so no cache has to be written back or dropped as a whole; the
// compiler is held to the order "partial tile, ticket" and "last ticket, reads" by a release and
// an acquire fence at workgroup scope around them (tzgemm_role_ksplit).
// A partial tile is 16 blocks of 64 x float4 (block = i * 4 + j of the accumulator set),
// stored as two 8-byte halves per lane: [block][half][lane].
typedef unsigned long long tz_u64;
__device__ __forceinline__ void tz_partial_store(tz_u64 *tile, int block, int lane, float4_t v)
{
    union { float4_t f; tz_u64 q[2]; } u;
    u.f = v;
    __hip_atomic_store(tile + (block * 2 + 0) * 64 + lane, u.q[0], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(tile + (block * 2 + 1) * 64 + lane, u.q[1], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float4_t tz_partial_load(const tz_u64 *tile, int block, int lane)
{
    union { float4_t f; tz_u64 q[2]; } u;
    u.q[0] = __hip_atomic_load(tile + (block * 2 + 0) * 64 + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    u.q[1] = __hip_atomic_load(tile + (block * 2 + 1) * 64 + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return u.f;
}

// B_ONCE: every row of B is read by one tile only -- a batch padded up to M = 128, of which the one tile
// row that holds the batch is launched: the weights of a fully connected layer -- so its loads carry the
// nontemporal hint and the weights pass by the caches instead of through them.  Per query that is 205 MB
// (fc1) that no longer push the next layers' operands and the co-located kernel's data out; measured
// with 512 MiB written before each launch: fc1 88.7 -> 55.9 us, fc2 23.4 -> 17.1 us.  (Launched back to
// back, where the previous launch's weights still sit in the memory-side cache, the hint costs:
// 35.7 -> 43.6 us -- not a state a query ever finds.)
template <bool B_ONCE, class Sync>
__device__ __forceinline__ void tzgemm_role_ksplit(const _Float16 *__restrict__ A,
                                                   const _Float16 *__restrict__ B, float *__restrict__ C,
                                                   int M, int N, int K, unsigned *workspace,
                                                   int role_block, int role_blocks, int tile_start,
                                                   int tile_end, int tid, char *lds, Sync &sync)
{
    typedef __attribute__((address_space(3))) void *lptr_t;
    constexpr int BK = TZ_BLOCK_K;
    constexpr int ROWB = BK * 2;                      // 128-byte tile rows
    constexpr int OPERAND_BYTES = TZ_REF_TILE * ROWB; // 8 KiB: 64 rows of one operand
    constexpr int STAGE = 2 * OPERAND_BYTES;          // A rows then B rows
    constexpr int LOADS = 8;                          // LDS-direct loads per operand and chunk
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int ref_cols = N / TZ_REF_TILE;
    const int n_ref = (M / TZ_REF_TILE) * ref_cols;
    const int kchunks = K / BK;
    const int parts = tz_ksplit_parts(M, N, K);
    tz_u64 *partial_tiles =
        reinterpret_cast<tz_u64 *>(reinterpret_cast<char *>(workspace) + tz_workspace_counter_bytes(M, N));
    char *mine = lds + wave * (2 * STAGE);            // this wave's two stages
    const unsigned mine_lds = (unsigned)(size_t)(lptr_t)mine;
    // load j of an operand fills rows 8j .. 8j+7: lane lands in row 8j + lane/8, slot lane%8,
    // and fetches the row's segment slot ^ ((row>>1)&7) = slot ^ (lane>>4) ^ (4*(j&1))
    const unsigned seg_even = (unsigned)((lane & 7) ^ (lane >> 4));
    const unsigned src_even = (unsigned)((lane >> 3) * K + (int)seg_even * 8) * 2u;
    const unsigned src_odd = (unsigned)((lane >> 3) * K + (int)(seg_even ^ 4u) * 8) * 2u;
    const int frag_key = ((lane & 15) >> 1) & 7;
    const int frag_seg0 = ((lane >> 4) ^ frag_key) * 16;
    const int frag_seg1 = ((4 + (lane >> 4)) ^ frag_key) * 16;
    const int frag_row = (lane & 15) * ROWB;
    if (tile_end > n_ref) tile_end = n_ref;
    if (parts > 1 && workspace == nullptr) {
        // the host binds one to every C it builds a kernel object on; a launch that reaches this
        // point without one computes nothing and says so (TK_FAIL_WORKSPACE), it never faults
        if (tid == 0 && role_block == 0)
            __hip_atomic_fetch_or(&tk_spin_fail, TK_FAIL_WORKSPACE, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        tile_end = tile_start;
    }
    const int tiles = tile_end - tile_start;
    const int units = tiles > 0 ? tiles * parts : 0;

    for (int round_base = 0; round_base < units; round_base += role_blocks) {
        const int in_round = tz_ksplit_unit_of(role_block, role_blocks, min(units - round_base, role_blocks));
        if (in_round < 0) break;
        const int unit = round_base + in_round;
        const int part = unit / tiles;
        const int pos = tile_start + unit % tiles;
        const int ti = pos / ref_cols;
        const int tj = pos % ref_cols;
        const int part_first = (part * kchunks) / parts;
        const int part_chunks = ((part + 1) * kchunks) / parts - part_first;
        const int c_first = part_first + (wave * part_chunks) / 4;
        const int c_last = part_first + ((wave + 1) * part_chunks) / 4;
        const char *a_tile = reinterpret_cast<const char *>(A + (size_t)(ti * TZ_REF_TILE) * K);
        const char *b_tile = reinterpret_cast<const char *>(B + (size_t)(tj * TZ_REF_TILE) * K);
#define TZK_ISSUE(chunk_, stage_)                                                                  \
    _Pragma("unroll") for (int j = 0; j < LOADS; ++j)                                              \
    {                                                                                              \
        const unsigned dst_ = mine_lds + (stage_) * STAGE + j * 1024;                              \
        const size_t uni_ = ((size_t)(j * 8) * K + (size_t)(chunk_) * BK) * 2;                     \
        const unsigned lane_ = (j & 1) ? src_odd : src_even;                                       \
        tz_load_to_lds(a_tile + uni_, lane_, dst_);                                                \
        if constexpr (B_ONCE) tz_load_to_lds_once(b_tile + uni_, lane_, dst_ + OPERAND_BYTES);     \
        else tz_load_to_lds(b_tile + uni_, lane_, dst_ + OPERAND_BYTES);                           \
    }
        float4_t acc[4][4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};
        if (c_first < c_last) { TZK_ISSUE(c_first, 0) }
        for (int c = c_first; c < c_last; ++c) {
            const int stage = (c - c_first) & 1;
            if (c + 1 < c_last) {
                TZK_ISSUE(c + 1, stage ^ 1)
                __builtin_amdgcn_s_waitcnt(TK_VMCNT_IMM(2 * LOADS));   // chunk c has landed
            } else {
                __builtin_amdgcn_s_waitcnt(TK_VMCNT_IMM(0));
            }
            half8_t fa[2][4], fb[2][4];
            const char *st = mine + stage * STAGE + frag_row;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                fa[0][i] = *reinterpret_cast<const half8_t *>(st + i * 16 * ROWB + frag_seg0);
                fb[0][i] = *reinterpret_cast<const half8_t *>(st + OPERAND_BYTES + i * 16 * ROWB + frag_seg0);
                fa[1][i] = *reinterpret_cast<const half8_t *>(st + i * 16 * ROWB + frag_seg1);
                fb[1][i] = *reinterpret_cast<const half8_t *>(st + OPERAND_BYTES + i * 16 * ROWB + frag_seg1);
            }
#pragma unroll
            for (int h = 0; h < 2; ++h)
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb[h][j], fa[h][i], acc[i][j], 0, 0, 0);
            // the reads above have returned (the MFMAs consumed them) before the next
            // iteration's loads overwrite this stage
            __builtin_amdgcn_s_waitcnt(TK_LGKMCNT0_IMM);
        }
#undef TZK_ISSUE
        // partial tiles of waves 1..3 go to LDS (each into its own region), wave 0 adds them
        if (wave != 0) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    *reinterpret_cast<float4_t *>(mine + ((i * 4 + j) * 64 + lane) * 16) = acc[i][j];
        }
        sync.sync();
        if (wave == 0) {
#pragma unroll
            for (int w = 1; w < 4; ++w)
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        acc[i][j] += *reinterpret_cast<const float4_t *>(lds + w * (2 * STAGE) +
                                                                         ((i * 4 + j) * 64 + lane) * 16);
            if (parts == 1) {
                float *c_lane = C + (size_t)(ti * TZ_REF_TILE + (lane & 15)) * N + tj * TZ_REF_TILE + (lane >> 4) * 4;
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        float4_t v = acc[i][j] * TZ_ALPHA;
                        *reinterpret_cast<float4_t *>(c_lane + (size_t)(i * 16) * N + j * 16) = v;
                    }
            } else {
                tz_u64 *my_partial = partial_tiles + ((size_t)pos * parts + part) * (TZ_PARTIAL_TILE_BYTES / 8);
                const int lane_here = tz_opaque(lane);
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int j = 0; j < 4; ++j) tz_partial_store(my_partial, i * 4 + j, lane_here, acc[i][j]);
                // The partial tile before the ticket.  For the hardware: the stores above are agent-scope
                // accesses (written through to the memory side all XCDs share) and the wave waits until
                // every one of them has been acknowledged.  For the compiler: a release fence, so that no
                // store can sink below the ticket.  The fence is at workgroup scope on purpose: at agent
                // scope it is a write-back of the XCD's whole L2 (buffer_wbl2), 1 to 2 us on a layer of
                // 11 to 14 us, for stores that have already left the L2.
                __builtin_amdgcn_s_waitcnt(TK_VMCNT_IMM(0));
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
                unsigned ticket = 0;
                if (lane == 0)
                    ticket = __hip_atomic_fetch_add(workspace + pos, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
                ticket = __builtin_amdgcn_readfirstlane(ticket);
                // tell every wave whether this workgroup drew the last ticket: one word at the head of
                // each wave's own LDS region (wave 0 is done with the partial tiles that were there)
                if (lane < 4)
                    *reinterpret_cast<unsigned *>(lds + lane * (2 * STAGE)) = (ticket == (unsigned)(parts - 1)) ? 1u : 0u;
            }
        }
        sync.sync();   // wave 0 has read the partial tiles before the next tile's loads land on them
        if (parts > 1 &&
            __builtin_amdgcn_readfirstlane(*(const __attribute__((address_space(3))) unsigned *)(lptr_t)mine) != 0u) {
            // last to arrive: add the partial tiles in part order.  Wave w takes rows 16w .. 16w+15 of
            // the tile; loads go out two parts at a time so that a batch is one trip to memory.
            // The ticket before the reads.  Wave 0 drew the last ticket and told the others through LDS
            // and the role barrier; every wave reads other workgroups' partial tiles itself.  For the
            // compiler: an acquire fence, so that no load can rise above the flag.  For the hardware:
            // the loads are agent-scope accesses of their own, which are served from the memory side,
            // not from a line this XCD's L2 may hold.  At agent scope the fence is an invalidation of
            // the whole L2 (buffer_inv), 5 to 6 us a layer.
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
            const tz_u64 *tile_parts = partial_tiles + (size_t)pos * parts * (TZ_PARTIAL_TILE_BYTES / 8);
            const int lane_here = tz_opaque(lane);
            float4_t sum[4];
            for (int p0 = 0; p0 < parts; p0 += TZ_KSPLIT_PARTS_IN_FLIGHT) {
                float4_t got[TZ_KSPLIT_PARTS_IN_FLIGHT][4];
#pragma unroll
                for (int q = 0; q < TZ_KSPLIT_PARTS_IN_FLIGHT; ++q)
                    if (p0 + q < parts) {
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            got[q][j] = tz_partial_load(tile_parts + (p0 + q) * (TZ_PARTIAL_TILE_BYTES / 8),
                                                        wave * 4 + j, lane_here);
                    }
#pragma unroll
                for (int q = 0; q < TZ_KSPLIT_PARTS_IN_FLIGHT; ++q)
                    if (p0 + q < parts) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) sum[j] = (p0 + q == 0) ? got[q][j] : sum[j] + got[q][j];
                    }
            }
            float *c_lane = C + (size_t)(ti * TZ_REF_TILE + wave * 16 + (lane & 15)) * N + tj * TZ_REF_TILE + (lane >> 4) * 4;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float4_t v = sum[j] * TZ_ALPHA;
                *reinterpret_cast<float4_t *>(c_lane + j * 16) = v;
            }
            if (tid == 0) __hip_atomic_store(workspace + pos, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        __builtin_amdgcn_s_waitcnt(TK_VMCNT_IMM(0));
    }
    sync.finish();
}

template <int STAGES, bool STREAM_C = true, class Sync>
__device__ __forceinline__ void tzgemm_role(const _Float16 *__restrict__ A, const _Float16 *__restrict__ B,
                                            float *__restrict__ C, int M, int N, int K, unsigned *workspace,
                                            int role_block, int role_blocks, int tile_start, int tile_end,
                                            int tid, char *lds, Sync &sync)
{
    static_assert(STAGES * TZ_STAGE_BYTES >= TZ_KSPLIT_LDS_BYTES,
                  "the K-split form needs two 16 KiB stages per wave");
    if (tz_use_ksplit(M, N, K)) {
        if (M == TZ_MACRO_TILE)
            tzgemm_role_ksplit<true>(A, B, C, M, N, K, workspace, role_block, role_blocks, tile_start, tile_end, tid,
                                     lds, sync);
        else
            tzgemm_role_ksplit<false>(A, B, C, M, N, K, workspace, role_block, role_blocks, tile_start, tile_end, tid,
                                      lds, sync);
    } else
        tzgemm_role_tiles<STAGES, STREAM_C>(A, B, C, M, N, K, role_block, role_blocks, tile_start, tile_end, tid, lds,
                                            sync);
}

// Workgroups of a launch of role_blocks that can hold a tile of this GEMM (the first ones, in
// both forms).  A fused kernel uses it to keep best-effort blocks off those workgroups when the
// GEMM leaves most of the chip without a tile.
__device__ __forceinline__ int tz_busy_workgroups(int M, int N, int K, int role_blocks, int tile_start,
                                                  int tile_end)
{
    if (tile_start >= tile_end) return 0;
    const int units = tz_use_ksplit(M, N, K) ? (tile_end - tile_start) * tz_ksplit_parts(M, N, K)
                                             : (M / TZ_MACRO_TILE) * (N / TZ_MACRO_TILE);
    return min(units, role_blocks);
}

}  // namespace tk
