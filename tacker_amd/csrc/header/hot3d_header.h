// hotspot3D constants (src/header/hot3d_header.h:9-24 of the reference; chip geometry and material
// constants of Rodinia's 3D thermal simulation).
#pragma once
#include "pets_common.h"
#define HOT3D_TILE_X 64       // block_dimension_x of the ori launch (src/ori_kernel/hot3d_kernel.cu:129)
#define HOT3D_TILE_Y 4        // block_dimension_y
#define HOT3D_AMB_TEMP 80.0f  // ambient temperature the top layer exchanges heat with
#define HOT3D_MAX_PD 3.0e6
#define HOT3D_PRECISION 0.001
#define HOT3D_SPEC_HEAT_SI 1.75e6
#define HOT3D_K_SI 100
#define HOT3D_FACTOR_CHIP 0.5
#define HOT3D_T_CHIP 0.0005f
#define HOT3D_CHIP_HEIGHT 0.016f
#define HOT3D_CHIP_WIDTH 0.016f
