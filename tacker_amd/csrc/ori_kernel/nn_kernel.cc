#include "nn_kernel.h"

#include <unordered_map>

#include "../Logger.h"
#include "fill.h"

extern Logger logger;
extern std::unordered_map<std::string, void *> fmap;

int nnBlocks(int numRecords) { return numRecords <= 0 ? 0 : (numRecords - 1) / NN_THREADS_PER_BLOCK + 1; }

OriNNKernel::OriNNKernel(int id)
{
    Id = id;
    this->kernelName = "nn";
    initParams();
}

OriNNKernel::OriNNKernel(int id, LatLong *d_locations, float *d_distances, int numRecords, float lat, float lng)
{
    Id = id;
    this->kernelName = "nn";
    NNKernelParams = new OriNNParamsStruct{d_locations, d_distances, numRecords, lat, lng};
    bind();
}

OriNNKernel::~OriNNKernel()
{
    for (auto &ptr : cudaFreeList) tkErrCheck(tkFree(ptr));
    delete NNKernelParams;
}

void OriNNKernel::initParams()
{
    const int numRecords = 256 * 2560000;
    LatLong *d_locations = nullptr;
    float *d_distances = nullptr;
    TK_SAFE_CALL(tkMalloc((void **)&d_locations, sizeof(LatLong) * (size_t)numRecords));
    cudaFreeList.push_back(d_locations);
    TK_SAFE_CALL(tkMalloc((void **)&d_distances, sizeof(float) * (size_t)numRecords));
    cudaFreeList.push_back(d_distances);
    // {lat, lng} interleaved: one fill over the 2 n floats
    tkFillUniform(reinterpret_cast<float *>(d_locations), 2 * (size_t)numRecords, 4001u, 0.0f, 90.0f);
    TK_SAFE_CALL(tkMemset(d_distances, 0, sizeof(float) * (size_t)numRecords));
    NNKernelParams = new OriNNParamsStruct{d_locations, d_distances, numRecords, 30.0f, 90.0f};
    bind();
}

void OriNNKernel::bind()
{
    if (NNKernelParams->numRecords <= 0) logger.ERROR("nn: at least one record");
    // the reference folds the blocks over gridDim.y only beyond maxGridSize[0] = 2^31 - 1 blocks
    // (src/ori_kernel/nn_kernel.cu:74-78), which an int record count never reaches
    launchGridDim = dim3((unsigned)nnBlocks(NNKernelParams->numRecords), 1, 1);
    launchBlockDim = dim3(NN_THREADS_PER_BLOCK, 1, 1);
    kernelParams = {&NNKernelParams->d_locations, &NNKernelParams->d_distances, &NNKernelParams->numRecords,
                    &NNKernelParams->lat, &NNKernelParams->lng};
    this->smem = 0;
    auto it = fmap.find("ori_nn");
    this->kernelFunc = it == fmap.end() ? nullptr : it->second;
    this->initialized = true;
}

void OriNNKernel::executeImpl(cudaStream_t stream)
{
    if (!kernelFunc) logger.ERROR("load kernel {ori_nn} failed!");
    TK_SAFE_CALL(tkLaunchKernel(this->kernelFunc, launchGridDim.raw(), launchBlockDim.raw(),
                                (void **)this->kernelParams.data(), 0, stream));
}
