// OriFFTKernel -- host object of Parboil's batched 256-point FFT
// (src/ori_kernel/fft_kernel.{h,cu} of the reference).
#pragma once
#include "../Kernel.h"
#include "../header/fft_header.h"

struct OriFFTParamsStruct {
    float *data;   // batches x 256 complex values (re, im), transformed in place
};

class OriFFTKernel : public Kernel {
public:
    // FFT_B = 10240 transforms of values uniform in [-1, 1) from rand() seeded with 54321
    // (src/ori_kernel/fft_kernel.cu:87-131; the reference allocates ten times the bytes it uses)
    explicit OriFFTKernel(int id);
    // caller-owned batch
    OriFFTKernel(int id, float *data, int batches);
    ~OriFFTKernel() override;

    void initParams() override;
    std::vector<int> getArgs() override { return std::vector<int>(); }
    OriFFTParamsStruct *params() { return FFTKernelParams; }

protected:
    void executeImpl(cudaStream_t stream) override;

private:
    void loadKernel() override {}
    void bind(int batches);
    OriFFTParamsStruct *FFTKernelParams = nullptr;
};
