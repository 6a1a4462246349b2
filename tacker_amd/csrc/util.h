// util.h -- host-side helpers shared by the runtime classes.
//
// Stands where src/util.h of the reference stands: the error-check macros the
// Kernel classes use, plus the launch-geometry types.  The reference includes
// the CUDA headers here; this runtime talks to the device only through the tk*
// C layer (include/tacker_amd.h), so the host classes compile with a plain C++
// compiler and can be linked against either the HIP implementation or the
// recording fake.
#pragma once

#include <cstdio>
#include <cstdlib>
#include <sstream>
#include <stdexcept>
#include <string>

#include "../../include/tacker_amd.h"

// dim3 as the reference's callers write it: dim3(x), dim3(x, y, z).
struct dim3 {
    unsigned x, y, z;
    dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
    tkDim3 raw() const { return tkDim3{x, y, z}; }
};

typedef tkStream_t cudaStream_t;   // the name the reference's signatures use
typedef tkFunction_t CUfunction;

// Runtime-API failure -> std::runtime_error with file and line
// (CUDA_SAFE_CALL, src/util.h:50-62).
#define TK_SAFE_CALL(x)                                                                        \
    do {                                                                                       \
        int tk_result_ = (x);                                                                  \
        if (tk_result_ != TK_SUCCESS) {                                                        \
            std::stringstream safe_call_ss;                                                    \
            safe_call_ss << "\nerror: " #x " failed with error"                                \
                         << "\nfile: " << __FILE__ << "\nline: " << __LINE__                   \
                         << "\nmsg: " << tkGetErrorString(tk_result_);                         \
            throw std::runtime_error(safe_call_ss.str());                                      \
        }                                                                                      \
    } while (0)

// Module (driver-style) failure -> message and exit (CU_SAFE_CALL, src/util.h:25-36).
#define TK_MODULE_SAFE_CALL(x)                                                                 \
    do {                                                                                       \
        int tk_result_ = (x);                                                                  \
        if (tk_result_ != TK_SUCCESS) {                                                        \
            fprintf(stderr, "TK_MODULE_SAFE_CALL() error = %04d \"%s\" from file <%s>, line %i.\n", \
                    tk_result_, tkGetErrorString(tk_result_), __FILE__, __LINE__);             \
            exit(EXIT_FAILURE);                                                                \
        }                                                                                      \
    } while (0)

// Allocation helpers print and continue (cudaErrCheck, src/util.h:65-70).
#define tkErrCheck(stat)                                                                       \
    do {                                                                                       \
        int tk_result_ = (stat);                                                               \
        if (tk_result_ != TK_SUCCESS)                                                          \
            fprintf(stderr, "TK Error: %s %s %d\n", tkGetErrorString(tk_result_), __FILE__,    \
                    __LINE__);                                                                 \
    } while (0)
