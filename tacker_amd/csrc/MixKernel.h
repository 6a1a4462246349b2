// MixKernel.h -- one fused launch of two GPTB kernels.
//
// Same contract as src/MixKernel.h of the reference: the parameter vector is
// [kernel1 params + 6 dims][start1, step1, end1][kernel2 params + 6 dims]
// [start2, step2, end2]; both steps equal the fused launch's grid size; the
// device function is looked up in the registry under funcKey; the vectors of the
// two GPTB kernels are copied at construction (later edits of their ranges are
// not seen).  smem stays 0: fused kernels declare their LDS statically.
#pragma once

#include "GPTBKernel.h"
#include "json.h"

extern Logger logger;
extern std::unordered_map<std::string, void *> fmap;

class MixKernel : public Kernel {
public:
    MixKernel(int id, const std::string &funcKey, GPTBKernel *kernel1, GPTBKernel *kernel2,
              dim3 gridDim, dim3 blockDim, int ptb_start_block_pos1, int ptb_end_block_pos1,
              int ptb_start_block_pos2, int ptb_end_block_pos2)
        : funcKey(funcKey), kernel1(kernel1), kernel2(kernel2)
    {
        this->Id = id;
        this->kernelName = funcKey;
        this->launchGridDim = gridDim;
        this->launchBlockDim = blockDim;
        this->smem = 0;

        const int step = (int)(gridDim.x * gridDim.y * gridDim.z);
        kernel1_start_block_pos = ptb_start_block_pos1;
        kernel1_iter_block_step = step;
        kernel1_end_block_pos = ptb_end_block_pos1;
        kernel2_start_block_pos = ptb_start_block_pos2;
        kernel2_iter_block_step = step;
        kernel2_end_block_pos = ptb_end_block_pos2;

        initParams();
        loadKernel();
    }

    const std::string funcKey;

    int kernel1_start_block_pos;
    int kernel1_iter_block_step;
    int kernel1_end_block_pos;
    int kernel2_start_block_pos;
    int kernel2_iter_block_step;
    int kernel2_end_block_pos;

    void initParams() override
    {
        kernelParams.insert(kernelParams.end(), kernel1->kernelParams.begin(), kernel1->kernelParams.end());
        kernelParams.push_back(&kernel1_start_block_pos);
        kernelParams.push_back(&kernel1_iter_block_step);
        kernelParams.push_back(&kernel1_end_block_pos);
        kernelParams.insert(kernelParams.end(), kernel2->kernelParams.begin(), kernel2->kernelParams.end());
        kernelParams.push_back(&kernel2_start_block_pos);
        kernelParams.push_back(&kernel2_iter_block_step);
        kernelParams.push_back(&kernel2_end_block_pos);
    }

    void loadKernel() override
    {
        auto it = fmap.find(funcKey);
        if (it == fmap.end()) logger.ERROR("load kernel {" + funcKey + "} failed!");
        this->kernelFunc = it->second;
    }

    std::vector<int> getArgs() override { return std::vector<int>(); }

protected:
    void executeImpl(cudaStream_t stream) override
    {
        TK_SAFE_CALL(launchBy((void **)kernelParams.data(), stream));
    }

private:
    GPTBKernel *kernel1;
    GPTBKernel *kernel2;
};
