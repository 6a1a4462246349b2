// 7-point stencil constants (src/header/stencil_header.h of the reference).
#pragma once
#include "pets_common.h"
#define STENCIL_TILE_X 32     // block_dimension_x of the ori launch; 2 points per thread in x
#define STENCIL_TILE_Y 4      // block_dimension_y
#define Index3D(_nx, _ny, _i, _j, _k) ((_i) + (_nx) * ((_j) + (_ny) * (_k)))
// centre planes of one run of the z march: the unit a block column is cut into along z
// (grid_dimension_z of the GPTB position space counts these runs)
#define STENCIL_Z_RUN 8
