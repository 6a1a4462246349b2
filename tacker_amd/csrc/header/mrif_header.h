// MRI-FHD constants (src/header/mrif_header.h of the reference).
#pragma once
#include "pets_common.h"
#define KERNEL_RHO_PHI_THREADS_PER_BLOCK 256
#define KERNEL_FH_THREADS_PER_BLOCK 256
#define KERNEL_FH_K_ELEMS_PER_GRID 256
#define MRIF_MAX_K 4096          // capacity of the constant k table (80 KiB)
// k records one block position of the GPTB form adds to its 256 voxels
#define MRIF_K_CHUNK 128
struct mrif_kValues {
    float Kx;
    float Ky;
    float Kz;
    float RhoPhiR;
    float RhoPhiI;
};
