// OriSTENCILKernel -- host object of the 7-point stencil
// (src/ori_kernel/stencil_kernel.{h,cu} of the reference).
#pragma once
#include "../Kernel.h"

struct OriSTENCILParamsStruct {
    float c0;
    float c1;
    float *A0;
    float *Anext;
    int nx;
    int ny;
    int nz;
};

class OriSTENCILKernel : public Kernel {
public:
    // allocates A0/Anext for 512x512x64, fills A0 with seeded uniform[0,1), Anext = A0
    explicit OriSTENCILKernel(int id);
    // caller-owned grids of any size
    OriSTENCILKernel(int id, float c0, float c1, const float *A0, float *Anext, int nx, int ny, int nz);
    ~OriSTENCILKernel() override;

    void initParams() override;
    std::vector<int> getArgs() override { return std::vector<int>(); }
    // exchange A0 and Anext (one Jacobi iteration done; Parboil's pointer swap)
    void swapGrids();
    OriSTENCILParamsStruct *params() { return STENCILKernelParams; }

protected:
    void executeImpl(cudaStream_t stream) override;

private:
    void loadKernel() override {}
    void bind();
    OriSTENCILParamsStruct *STENCILKernelParams = nullptr;
    bool ownsBuffers = false;
};
