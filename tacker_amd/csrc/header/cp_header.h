// Coulomb-potential constants (src/header/cp_header.h of the reference).
#pragma once
#include "pets_common.h"
#define BLOCKSIZEX 16
#define BLOCKSIZEY 8
#define UNROLLX 8
#define MAXATOMS 64
#define VOLSIZEX 4096
#define VOLSIZEY 4096
#define ATOMCOUNT 4000
// x points of a thread that one block position of the GPTB form computes, and the
// positions a block is made of (the switch in cp_role lists the parts: keep it at 4)
#define CP_POINTS_PER_POSITION 2
#define CP_X_PARTS (UNROLLX / CP_POINTS_PER_POSITION)
