#include "fft_kernel.h"

#include <cstdlib>
#include <unordered_map>
#include <vector>

#include "../Logger.h"

extern Logger logger;
extern std::unordered_map<std::string, void *> fmap;

OriFFTKernel::OriFFTKernel(int id)
{
    Id = id;
    this->kernelName = "fft";
    initParams();
}

OriFFTKernel::OriFFTKernel(int id, float *data, int batches)
{
    Id = id;
    this->kernelName = "fft";
    FFTKernelParams = new OriFFTParamsStruct{data};
    bind(batches);
}

OriFFTKernel::~OriFFTKernel()
{
    for (auto &ptr : cudaFreeList) tkErrCheck(tkFree(ptr));
    delete FFTKernelParams;
}

void OriFFTKernel::initParams()
{
    const size_t values = (size_t)FFT_N * FFT_B * 2;
    std::vector<float> source(values);
    srand(54321);
    for (size_t i = 0; i < values; ++i) source[i] = (rand() / (float)RAND_MAX) * 2 - 1;   // x then y of each point
    float *data = nullptr;
    TK_SAFE_CALL(tkMalloc((void **)&data, values * sizeof(float)));
    cudaFreeList.push_back(data);
    TK_SAFE_CALL(tkMemcpy(data, source.data(), values * sizeof(float), TK_MEMCPY_H2D));
    FFTKernelParams = new OriFFTParamsStruct{data};
    bind(FFT_B);
}

void OriFFTKernel::bind(int batches)
{
    if (batches <= 0) logger.ERROR("fft: the batch must hold at least one transform");
    // one block position per transform (src/ori_kernel/fft_kernel.cu:112-115: grid FFT_B); a
    // wavefront serves it where the reference launches FFT_T = 128 threads
    launchGridDim = dim3(batches, 1, 1);
    launchBlockDim = dim3(FFT_WAVE, 1, 1);
    kernelParams = {&FFTKernelParams->data};
    this->smem = 0;
    auto it = fmap.find("ori_fft");
    this->kernelFunc = it == fmap.end() ? nullptr : it->second;
    this->initialized = true;
}

void OriFFTKernel::executeImpl(cudaStream_t stream)
{
    if (!kernelFunc) logger.ERROR("load kernel {ori_fft} failed!");
    TK_SAFE_CALL(tkLaunchKernel(this->kernelFunc, launchGridDim.raw(), launchBlockDim.raw(),
                                (void **)this->kernelParams.data(), 0, stream));
}
