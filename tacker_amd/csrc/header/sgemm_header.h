// SGEMM constants (src/header/sgemm_header.h of the reference: TILE_N 16, TILE_TB_HEIGHT 8,
// TILE_M = TILE_N * TILE_TB_HEIGHT; alpha = beta = 2 are literals of the kernel,
// src/ori_kernel/sgemm_kernel.cu:14-15).
#pragma once
#include "pets_common.h"
#define SGEMM_TILE_N 16
#define SGEMM_TILE_TB_HEIGHT 8
#define SGEMM_TILE_M (SGEMM_TILE_N * SGEMM_TILE_TB_HEIGHT)   // 128 rows of C per block, one per thread
#define SGEMM_ALPHA 2.0f
#define SGEMM_BETA 2.0f
// k steps one block position of the GPTB form adds to its 128 x 16 partial results
#define SGEMM_K_CHUNK 64
