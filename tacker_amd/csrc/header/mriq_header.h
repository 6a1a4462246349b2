// MRI-Q constants (src/header/mriq_header.h of the reference).
#pragma once
#include "pets_common.h"
#define PIx2_MRIQ 6.2831853071795864769252867665590058f
#define KERNEL_PHI_MAG_THREADS_PER_BLOCK 512
#define KERNEL_Q_THREADS_PER_BLOCK 256
#define KERNEL_Q_K_ELEMS_PER_GRID 1024
#define MRIQ_MAX_K 4096          // capacity of the constant k table (64 KiB)
// k records one block position of the GPTB form adds to its 256 voxels
#define MRIQ_K_CHUNK 128
struct mriq_kValues {
    float Kx;
    float Ky;
    float Kz;
    float PhiMag;
};
