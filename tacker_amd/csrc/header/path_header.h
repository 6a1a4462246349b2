// pathfinder constants (src/header/path_header.h:7-17 of the reference).
#pragma once
#include "pets_common.h"
#define PATH_BLOCK_SIZE 256   // columns one block position works on, halo included
#define PATH_HALO 1
#define PATH_SEED 9           // M_SEED
// columns of a position a lane holds here: one wavefront serves a position
#define PATH_COLS_PER_LANE (PATH_BLOCK_SIZE / TK_WAVE_SIZE)
