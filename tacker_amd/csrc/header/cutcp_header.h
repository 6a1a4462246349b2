// Cutoff Coulomb potential constants (src/header/cutcp_header.h:2-14 of the reference).
#pragma once
#include "pets_common.h"
#define BIN_DEPTH 8           // atoms a bin can hold
#define BIN_SIZE 32           // floats of a bin: BIN_DEPTH x {x, y, z, q}
#define BIN_SHIFT 5
#define BIN_CACHE_MAXLEN 32   // bins the reference's block caches at a time
#define BIN_LENGTH 4.f        // edge of a bin, in Angstroms
#define BIN_INVLEN (1.f / BIN_LENGTH)
#define REGION_SIZE 512       // lattice points of a region: 8 x 8 x 8
#define NBRLIST_DIM 11
#define NBRLIST_MAXLEN (NBRLIST_DIM * NBRLIST_DIM * NBRLIST_DIM)
// threads of the reference's block (8, 2, 8): each takes 4 points of its region, 2 apart in y
#define CUTCP_BLOCK_THREADS 128
// bins of the neighbour list one block position of the GPTB form walks (the reference's block stages
// BIN_CACHE_MAXLEN bins at a time: the same granularity)
#define CUTCP_NBR_CHUNK BIN_CACHE_MAXLEN
