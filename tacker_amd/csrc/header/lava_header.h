// lavaMD constants and data layout (src/header/lava_header.h:5-68 of the reference): particles in
// boxes of NUMBER_PAR_PER_BOX, every box with the list of its up to 26 neighbours.
#pragma once
#include "pets_common.h"
#define NUMBER_PAR_PER_BOX 100
#define LAVA_MAX_NEIGHBOURS 26
// parts of a box's work in the GPTB position grid: the home box itself and each neighbour slot
#define LAVA_PARTS (1 + LAVA_MAX_NEIGHBOURS)

typedef struct {
    float x, y, z;
} THREE_VECTOR;

typedef struct {
    float v, x, y, z;
} FOUR_VECTOR;

typedef struct nei_str {
    int x, y, z;
    int number;
    long offset;
} nei_str;

typedef struct box_str {
    int x, y, z;
    int number;
    long offset;
    int nn;
    nei_str nei[LAVA_MAX_NEIGHBOURS];
} box_str;

typedef struct par_str {
    float alpha;
} par_str;

typedef struct dim_str {
    int cur_arg;
    int arch_arg;
    int cores_arg;
    int boxes1d_arg;
    long number_boxes;
    long box_mem;
    long space_elem;
    long space_mem;
    long space_mem2;
} dim_str;
