// OriLBMKernel -- host object of the D3Q19 lattice-Boltzmann step
// (src/ori_kernel/lbm_kernel.{h,cu} of the reference).
#pragma once
#include "../Kernel.h"

struct OriLBMParamsStruct {
    float *src;
    float *dst;
};

class OriLBMKernel : public Kernel {
public:
    // allocates two 120x120x150 grids (20 entry planes + the reference's margins),
    // seeds src with the rest equilibrium plus noise and ~5% obstacle cells
    explicit OriLBMKernel(int id);
    // caller-owned grids: src/dst point at entry plane 0 of cell (0,0,0)
    OriLBMKernel(int id, const float *src, float *dst, int sx, int sy, int sz);
    ~OriLBMKernel() override;

    void initParams() override;
    std::vector<int> getArgs() override { return std::vector<int>(); }
    void swapGrids();
    OriLBMParamsStruct *params() { return LBMKernelParams; }
    int sizeX() const { return sx_; }
    int sizeY() const { return sy_; }
    int sizeZ() const { return sz_; }

protected:
    void executeImpl(cudaStream_t stream) override;

private:
    void loadKernel() override {}
    void bind();
    OriLBMParamsStruct *LBMKernelParams = nullptr;
    int sx_ = 0, sy_ = 0, sz_ = 0;
};
