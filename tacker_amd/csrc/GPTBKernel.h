// GPTBKernel.h -- persistent-workgroup wrapper around an "ori" kernel object.
//
// Same contract as src/GPTBKernel.h of the reference: the wrapper aliases the
// wrapped kernel's parameter pointers, appends pointers to its own six
// grid/block dimension ints at construction, and at every launch temporarily
// appends start / step / end / thread_base (step = current launch grid size),
// launches funcKey's device function from the registry, and removes the four
// again -- so a MixKernel built from it sees only the 6-dimension form.  Not
// re-entrant and not thread-safe, as in the reference.
#pragma once

#include <string>
#include <unordered_map>

#include "Kernel.h"
#include "Logger.h"
#include "ModuleCenter.h"

extern Logger logger;
extern ModuleCenter moduleCenter;
extern std::unordered_map<std::string, void *> fmap;

class GPTBKernel : public Kernel {
public:
    // extraParams: optional array of 20 ints appended (by address) right after the
    // wrapped kernel's own parameters -- the reference's second constructor form.
    GPTBKernel(int id, const std::string kernelName, const std::string funcKey, Kernel *kernel,
               dim3 gridDim, dim3 blockDim, int ptb_start_block_pos, int ptb_end_block_pos,
               int *extraParams = nullptr)
        : funcKey(funcKey), kernel_(kernel)
    {
        this->Id = id;
        this->kernelName = kernelName;
        this->launchGridDim = gridDim;
        this->launchBlockDim = blockDim;

        gptbParams.grid_dimension_x = (int)kernel_->launchGridDim.x;
        gptbParams.grid_dimension_y = (int)kernel_->launchGridDim.y;
        gptbParams.grid_dimension_z = (int)kernel_->launchGridDim.z;
        gptbParams.block_dimension_x = (int)kernel_->launchBlockDim.x;
        gptbParams.block_dimension_y = (int)kernel_->launchBlockDim.y;
        gptbParams.block_dimension_z = (int)kernel_->launchBlockDim.z;
        gptbParams.ptb_start_block_pos = ptb_start_block_pos;
        gptbParams.ptb_iter_block_step = (int)(gridDim.x * gridDim.y * gridDim.z);
        gptbParams.ptb_end_block_pos = ptb_end_block_pos;

        this->kernelParams = kernel_->kernelParams;   // alias the wrapped object's storage
        if (extraParams)
            for (int i = 0; i < 20; i++) this->kernelParams.push_back((void *)&extraParams[i]);
        this->smem = kernel_->smem;
        loadKernel();
        initParams();
    }

    ~GPTBKernel() override
    {
        logger.DEBUG("kernel name: " + kernelName + ", id: " + std::to_string(Id) + " is destroyed!");
    }

    GPTBParams gptbParams;
    const std::string funcKey;
    Kernel *kernel_;

    void initParams() override
    {
        int *dims[6] = {&gptbParams.grid_dimension_x,  &gptbParams.grid_dimension_y,
                        &gptbParams.grid_dimension_z,  &gptbParams.block_dimension_x,
                        &gptbParams.block_dimension_y, &gptbParams.block_dimension_z};
        for (int *d : dims) kernelParams.push_back(d);
        // start/step/end stay off the vector so that MixKernel can append its own
    }

    void loadKernel() override
    {
        auto it = fmap.find(funcKey + kernel_->funcVariant());   // a build made for this problem, if any
        if (it == fmap.end()) it = fmap.find(funcKey);
        if (it == fmap.end()) logger.ERROR("load kernel {" + funcKey + "} failed!");
        this->kernelFunc = it->second;
    }

    std::vector<int> getArgs() override { return std::vector<int>(); }

protected:
    void executeImpl(cudaStream_t stream) override
    {
        gptbParams.ptb_iter_block_step = (int)(launchGridDim.x * launchGridDim.y * launchGridDim.z);
        int thread_base = 0;   // a plain GPTB launch has no thread offset
        const size_t base = kernelParams.size();
        kernelParams.push_back(&gptbParams.ptb_start_block_pos);
        kernelParams.push_back(&gptbParams.ptb_iter_block_step);
        kernelParams.push_back(&gptbParams.ptb_end_block_pos);
        kernelParams.push_back(&thread_base);
        const int launch_status = launchBy((void **)kernelParams.data(), stream);
        kernelParams.resize(base);   // also on failure: the vector must not keep &thread_base
        TK_SAFE_CALL(launch_status);
    }
};
