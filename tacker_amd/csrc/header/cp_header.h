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
