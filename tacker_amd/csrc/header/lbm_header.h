// D3Q19 lattice-Boltzmann constants (src/header/lbm_header.h of the reference).
// Grid extents are run-time values here (the reference fixes 128^3 by macro);
// the SoA layout, entry order, flags and relaxation constants are the same.
#pragma once
#include "pets_common.h"
enum LbmEntry { LBM_C = 0, LBM_N, LBM_S, LBM_E, LBM_W, LBM_T, LBM_B, LBM_NE, LBM_NW, LBM_SE,
                LBM_SW, LBM_NT, LBM_NB, LBM_ST, LBM_SB, LBM_ET, LBM_EB, LBM_WT, LBM_WB,
                LBM_FLAGS, LBM_N_CELL_ENTRIES };
enum LbmCellFlags { LBM_OBSTACLE = 1 << 0, LBM_ACCEL = 1 << 1, LBM_IN_OUT_FLOW = 1 << 2 };
#define LBM_OMEGA (1.95f)
#define LBM_DFL1 (1.0f / 3.0f)
#define LBM_DFL2 (1.0f / 18.0f)
#define LBM_DFL3 (1.0f / 36.0f)
// floats between the allocation base and entry plane 0 (REAL_MARGIN) and the
// padding the allocation carries at both ends (TOTAL_MARGIN)
#define LBM_REAL_MARGIN(sx, sy) (2L * (sx) * (sy))
#define LBM_TOTAL_MARGIN(sx, sy) (2L * (sx) * (sy) * LBM_N_CELL_ENTRIES)
