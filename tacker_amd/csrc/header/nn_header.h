// Nearest-neighbour constants and record layout (src/header/nn_header.h:12-25 of the reference).
#pragma once
#include "pets_common.h"
#define NN_THREADS_PER_BLOCK 256   // DEFAULT_THREADS_PER_BLOCK: records of one block position
typedef struct latLong {
    float lat;
    float lng;
} LatLong;
