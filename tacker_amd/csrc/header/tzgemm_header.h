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

#define TZ_ALPHA 1.1f             // alpha_g, src/header/tzgemm_header.h:64
