// FFT constants (src/header/fft_header.h:13-18 of the reference: 10240 batched 256-point complex
// transforms, radix 2, one block of FFT_N / FFT_R threads per transform).
#pragma once
#include "pets_common.h"
#define FFT_B 10240
#define FFT_N 256
#define FFT_R 2
#define FFT_T (FFT_N / FFT_R)
// threads that serve one transform here: one wavefront, every lane playing two of the reference's
// threads (j and j + 64)
#define FFT_WAVE 64
