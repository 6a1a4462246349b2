// tzgemm tile constants.
// The reference (src/header/tzgemm_header.h) describes a 64x64 CTA tile built
// from 16x16x16 WMMA fragments by 4 warps of 32.  Its tile is kept as the unit
// of the [start,end) range interface (TZ_REF_TILE); the gfx950 kernel computes a
// 128x128 macro tile (2x2 reference tiles) per 256-thread workgroup with
// v_mfma_f32_16x16x32_f16, one reference tile per 64-wide wavefront, fed by a
// ring of LDS stages that the global loads fill directly (no register staging).
#pragma once
#include "pets_common.h"

#define TZ_REF_TILE 64            // BLOCK_ROW_TILES * WMMA_N of the reference
#define TZ_MACRO_TILE 128         // rows and columns of C per workgroup
#define TZ_THREADS 256            // 4 wavefronts, 2x2 over the macro tile
#define TZ_MFMA_M 16
#define TZ_MFMA_N 16
#define TZ_MFMA_K 32
#define TZ_BLOCK_K 64             // K extent of one LDS stage (128-byte tile rows)
#define TZ_STAGE_BYTES (2 * TZ_MACRO_TILE * TZ_BLOCK_K * 2)   // A rows then B rows: 32 KiB
#define TZ_STAGES 4               // LDS ring depth where the GEMM has the CU's LDS to itself
#define TZ_STAGES_WG 4            // ring depth of workgroup-split fused kernels
// issue priority of the tzgemm waves of a wave-split fused kernel (s_setprio, 0..3)
#ifndef TK_GEMM_WAVE_PRIORITY
#define TK_GEMM_WAVE_PRIORITY 3
#endif
#define TZ_LDS_BYTES (TZ_STAGES * TZ_STAGE_BYTES)
#define TZ_LDS_BYTES_WG (TZ_STAGES_WG * TZ_STAGE_BYTES)

// shapes that take the K-split form of the kernel (one reference tile per workgroup, K cut
// over its 4 waves): few macro tiles for the CUs there are, and a reduction worth cutting
#define TZ_KSPLIT_MAX_MACRO_TILES 64
#define TZ_KSPLIT_MIN_K 512
#define TZ_KSPLIT_LDS_BYTES (4 * 2 * 2 * TZ_REF_TILE * TZ_BLOCK_K * 2)   // two 16 KiB stages per wave
// ... and, when the tiles are fewer still, the reduction of one tile is also cut over several
// workgroups ("parts"): each adds its share of K into a partial tile in the workspace, and the
// last one to finish adds the partial tiles in part order and stores C.
#define TZ_KSPLIT_TARGET_WORKGROUPS 256   // parts are chosen to give about this many workgroups a share
#define TZ_KSPLIT_MAX_PARTS 8
#define TZ_KSPLIT_MIN_CHUNKS_PER_PART 8   // TZ_BLOCK_K chunks: two per wave
#define TZ_PARTIAL_TILE_BYTES (TZ_REF_TILE * TZ_REF_TILE * 4)
#define TZ_KSPLIT_PARTS_IN_FLIGHT 2      // partial tiles the last workgroup loads at a time (registers)
#define TZ_WORKSPACE_ALIGN 1024

#ifdef __HIPCC__
#define TZ_HOST_DEVICE __host__ __device__
#else
#define TZ_HOST_DEVICE
#endif

// Both depend on (M, N, K) only -- never on the launch -- so a fused launch and the plain kernel
// always add in the same order.
TZ_HOST_DEVICE inline bool tz_use_ksplit(int M, int N, int K)
{
    const int n_macro = (M / TZ_MACRO_TILE) * (N / TZ_MACRO_TILE);
    return n_macro <= TZ_KSPLIT_MAX_MACRO_TILES && K >= TZ_KSPLIT_MIN_K;
}
// workgroups that share the reduction of one reference tile (1: no workspace needed)
TZ_HOST_DEVICE inline int tz_ksplit_parts(int M, int N, int K)
{
    if (!tz_use_ksplit(M, N, K)) return 1;
    const int n_ref = (M / TZ_REF_TILE) * (N / TZ_REF_TILE);
    // M at its minimum of 128 is a batch padded up (a fully-connected layer at batch 1 .. 64): the
    // caller launches the tile row that holds its batch, half of the tiles, and the parts are sized
    // for that half
    const int launched = M == TZ_MACRO_TILE ? n_ref / 2 : n_ref;
    int parts = TZ_KSPLIT_TARGET_WORKGROUPS / launched;
    const int by_k = (K / TZ_BLOCK_K) / TZ_KSPLIT_MIN_CHUNKS_PER_PART;
    if (parts > by_k) parts = by_k;
    if (parts > TZ_KSPLIT_MAX_PARTS) parts = TZ_KSPLIT_MAX_PARTS;
    return parts < 1 ? 1 : parts;
}
// Workspace of one GEMM: a zeroed arrival counter per reference tile (the kernel leaves them
// zero again), then parts partial tiles per reference tile.  0 when the shape needs none.
TZ_HOST_DEVICE inline long long tz_workspace_counter_bytes(int M, int N)
{
    const long long n_ref = (long long)(M / TZ_REF_TILE) * (N / TZ_REF_TILE);
    return (n_ref * 4 + TZ_WORKSPACE_ALIGN - 1) / TZ_WORKSPACE_ALIGN * TZ_WORKSPACE_ALIGN;
}
TZ_HOST_DEVICE inline long long tz_workspace_bytes(int M, int N, int K)
{
    const int parts = tz_ksplit_parts(M, N, K);
    if (parts == 1) return 0;
    const long long n_ref = (long long)(M / TZ_REF_TILE) * (N / TZ_REF_TILE);
    return tz_workspace_counter_bytes(M, N) + n_ref * parts * TZ_PARTIAL_TILE_BYTES;
}

// Shapes the stand-alone kernel computes with 256 x 256 macro tiles (kernels/tzgemm_large.h):
// whole 256 x 256 tiles and at least one of them for every CU.  Same bits as the other forms.
#define TZ_LARGE_TILE 256
#define TZ_LARGE_MIN_TILES TK_CU_NUM
// the large-tile form writes a C above this size with nontemporal stores
#define TZ_LARGE_STREAM_C_BYTES (128u << 20)
TZ_HOST_DEVICE inline bool tz_use_large(int M, int N, int K)
{
    (void)K;
    return M % TZ_LARGE_TILE == 0 && N % TZ_LARGE_TILE == 0 &&
           (long long)(M / TZ_LARGE_TILE) * (N / TZ_LARGE_TILE) >= TZ_LARGE_MIN_TILES;
}

// The GEMM role of a 512-thread fused kernel (variant wave_256_large) takes 256 x 128 tiles
// (tzgemm_role_large_rot) for every shape they divide -- whole tiles, an even number of 64-k steps --
// that is not one of the K-split forms', and the 128 x 128 form otherwise: tz_large_fused_fits, asked by the kernel.  The host picks that
// variant by itself only where it pays, a tile for every CU: tz_use_large_fused.
#define TZ_LARGE_FUSED_TILE_M 256
#define TZ_LARGE_FUSED_TILE_N 128
TZ_HOST_DEVICE inline bool tz_large_fused_fits(int M, int N, int K)
{
    // (not the shapes of the K-split forms: there the order of additions is another one, and a fused
    // launch gives the bits of the plain kernel whatever its form)
    return M % TZ_LARGE_FUSED_TILE_M == 0 && N % TZ_LARGE_FUSED_TILE_N == 0 && K % 128 == 0 && !tz_use_ksplit(M, N, K);
}
TZ_HOST_DEVICE inline bool tz_use_large_fused(int M, int N, int K)
{
    return tz_large_fused_fits(M, N, K) &&
           (long long)(M / TZ_LARGE_FUSED_TILE_M) * (N / TZ_LARGE_FUSED_TILE_N) >= TZ_LARGE_MIN_TILES;
}

// Where a kernel finds the workspace of the output buffer it writes: a device-resident hash
// table from C to workspace that the host fills when it binds one (open addressing, linear
// probing, an entry is never moved or removed while kernels may run; key 0 = empty).  The
// reference's tzgemm has no such buffer and its parameter list (A, B, C, M, N, K) has no slot for
// one, so the kernels look it up by the pointer they are given anyway.
#define TZ_WS_TABLE_SLOTS 1024
#define TZ_WS_TABLE_MAX_PROBES 16
struct tz_ws_entry {
    unsigned long long c;           // key (below), 0 = empty slot, TZ_WS_TOMBSTONE = a binding that was taken out
    unsigned long long workspace;   // its workspace
};
#define TZ_WS_TOMBSTONE 1ull
// Table keys of an output buffer C.  The two kinds of kernel that bind a workspace to their output
// (tzgemm's shared reductions, sgemm's k parts) use different keys, so that they never share one:
// an output buffer is at least 4-byte aligned, so C + 2 is no buffer's address.
TZ_HOST_DEVICE inline unsigned long long tz_ws_key_tzgemm(const void *C) { return (unsigned long long)(size_t)C; }
TZ_HOST_DEVICE inline unsigned long long tz_ws_key_sgemm(const void *C) { return (unsigned long long)(size_t)C + 2ull; }
TZ_HOST_DEVICE inline unsigned tz_ws_hash(unsigned long long c)
{
    return (unsigned)(((c >> 8) * 0x9E3779B97F4A7C15ull) >> 54) & (TZ_WS_TABLE_SLOTS - 1);
}
// the device array the no-allocation entry point uses as workspace: the largest one any shape
// needs (a batch padded to M = 128 with N = 8192: 256 tiles x 2 parts) plus the counters
#define TZ_SCRATCH_BYTES ((8u << 20) + (64u << 10))

// bits of the device word tk_spin_fail
#define TK_FAIL_SPIN 1u        // a role-local barrier gave up waiting
#define TK_FAIL_WORKSPACE 2u   // a GEMM whose reduction is shared by workgroups found no workspace for its C

#define TZ_ALPHA 1.1f             // alpha_g, src/header/tzgemm_header.h:64
