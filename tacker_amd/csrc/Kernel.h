// Kernel.h -- base of every launchable object of the runtime.
//
// Public surface of src/Kernel.h of the reference (Kernel, lmode, GPTBParams):
// same member names, same void*-per-argument parameter vector, same
// execute()/initParams()/loadKernel()/getArgs() protocol, so TaskManager, Task
// and Creator code written against the reference compiles against this.
// Launches go through tkLaunchKernel (HIP: hipLaunchKernel) instead of
// cudaLaunchKernel.
#pragma once

#include <string>
#include <utility>
#include <vector>

#include "util.h"

enum lmode { DRIVER_LAUNCH = 0, RUNTIME_LAUNCH };

class Kernel {
public:
    virtual ~Kernel() = default;

    // execute(stream): the one entry point callers use
    template <typename... Args>
    void execute(Args &&...args)
    {
        executeImpl(std::forward<Args>(args)...);
    }
    virtual void initParams() = 0;
    virtual void loadKernel() = 0;
    // integer description of the launch for the scheduler: {m,n,k} for a GEMM
    // (mixable == 1), the 14 convolution ints (mixable == 2), empty otherwise
    virtual std::vector<int> getArgs() = 0;

    // No counterpart in the reference.  Suffix a wrapper appends to its function key when it looks
    // the device function up ("" = the key as given): lets a kernel object pick among builds of
    // the same device function by what it knows about its problem, without its callers naming one.
    virtual const char *funcVariant() { return ""; }

    int getKernelId() { return Id; }
    std::string &getKernelName() { return kernelName; }

    // Switch this object to lmode DRIVER_LAUNCH: `function` is taken from the code object registered
    // with the ModuleCenter under `module` (the loadKernel of src/ori_kernel/cp_kernel.cu:423-434)
    // and launches go through tkModuleLaunchKernel (cuLaunchKernel) instead of the registry's
    // function.  false, and the object unchanged, when the module or the function is not there.
    bool useModule(const std::string &module, const std::string &function_name);

    int Id = 0;
    std::string kernelName;
    std::string moduleName;
    std::string funcKey;
    CUfunction function = nullptr;        // set when loaded through ModuleCenter
    unsigned int smem = 0;                // LDS bytes the device function declares
    std::vector<void *> kernelParams;     // one pointer per kernel argument, in order
    std::vector<void *> cudaFreeList;     // device buffers this object owns
    dim3 launchGridDim;
    dim3 launchBlockDim;
    lmode launchMode = RUNTIME_LAUNCH;
    void *kernelFunc = nullptr;           // registry value for tkLaunchKernel
    unsigned int mixable = 0;             // 0 solo only, 1 GEMM-shaped, 2 convolution-shaped
    bool initialized = false;

protected:
    virtual void executeImpl(cudaStream_t stream) = 0;
    // the launch of wrappers whose whole argument list is `params`: by the object's launch mode
    int launchBy(void **params, cudaStream_t stream)
    {
        if (launchMode == DRIVER_LAUNCH)
            return tkModuleLaunchKernel(function, launchGridDim.raw(), launchBlockDim.raw(), params, 0, stream);
        return tkLaunchKernel(kernelFunc, launchGridDim.raw(), launchBlockDim.raw(), params, 0, stream);
    }
};

// The uniform tail of every GPTB kernel's parameter list (thread_base follows
// and is supplied at launch time).
struct GPTBParams {
    int grid_dimension_x;
    int grid_dimension_y;
    int grid_dimension_z;
    int block_dimension_x;
    int block_dimension_y;
    int block_dimension_z;
    int ptb_start_block_pos;
    int ptb_iter_block_step;
    int ptb_end_block_pos;
};
