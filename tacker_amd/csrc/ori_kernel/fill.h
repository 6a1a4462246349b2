// Device-side fills for the large default instances of the Rodinia kernels: values that are a
// function of (index, seed) only, so a host restatement of tk_fill_value can name any element
// without the array ever existing on the host.
#pragma once
#include <cstddef>

// dst[i] = lo + (hi - lo) * u(i, seed), u in [0, 1) with 24 bits
void tkFillUniform(float *dst, size_t n, unsigned seed, float lo, float hi);
// dst[i] = h(i, seed) % mod
void tkFillIntMod(int *dst, size_t n, unsigned seed, int mod);
