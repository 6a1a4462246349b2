// VGG16 (batch 1, 224x224) as a latency-critical Task whose convolutions and
// fully-connected layers run on tzgemm.
//
// Stands where src/dnn/vgg16/ + src/include/dnn.h stand in the reference (a list
// of NNFusion-generated kernel objects whose convolutions are rerouted to
// im2col + ptb_tzgemm).  Kept: the Task / Kernel interface, mixable = 2 with the
// 14 convolution ints from getArgs() for conv layers, mixable = 1 with {m,n,k}
// for FC layers, so the TaskManager treats them exactly as the reference's.
// Different on purpose: the GEMMs consume the real activations and weights
// (random-initialised), dimensions are padded UP to multiples of 128 instead of
// floored, and a layer can be launched fused with a best-effort slice through
// LcGemmKernel::executeMixed.
#pragma once

#include <memory>
#include <string>
#include <vector>

#include "../GPTBKernel.h"
#include "../Task.h"
#include "../tzgemm_kernel.h"

// An LC kernel that is one tzgemm plus layer-specific data movement.
class LcGemmKernel : public Kernel {
public:
    // the layer with blocks [be_start, be_end) of a best-effort kernel fused into
    // its GEMM launch (be_end <= be_start: the GEMM alone)
    // variant: which generated form of the fused kernel ("" = the one kinfo names for the pair)
    virtual void executeMixed(GPTBKernel *be, int be_start, int be_end, cudaStream_t stream,
                              const std::string &variant = "") = 0;
    // padded GEMM shape {M, N, K} actually launched
    virtual std::vector<int> gemmDims() const = 0;
    void initParams() override {}
    void loadKernel() override {}
};

struct VGG16Options {
    int height = 224, width = 224;   // input resolution (multiples of 32)
    int classes = 1000;
    unsigned long long seed = 1337ULL;
};

class VGG16 : public Task {
public:
    explicit VGG16(int taskId, const VGG16Options &opt = VGG16Options());
    ~VGG16() override;
    void initExecution() override;       // host -> device copy of the input image
    // device pointer / length of the logits (column 0 of the last GEMM's output, stride ld)
    const float *logits(long *stride) const;
    // output buffer of layer `idx` (0..12 the convolutions, 13..15 the fully connected layers; for
    // tests): device pointer, rows, channel stride.  It holds 1.1 * A * B^T; bias (returned here,
    // none for the last layer) and ReLU are applied by the layer that reads it
    struct Act { float *ptr; int H, W, C, ld; void *weights; float *bias; int Np, Kp; };
    Act activation(int conv_index) const;
    VGG16Options opt;
    struct Impl;
    std::unique_ptr<Impl> impl;
};

// createTask (src/main.cu:227-244): the LC task by model name; unknown -> logger.ERROR
Task *createTask(const std::string &model);
