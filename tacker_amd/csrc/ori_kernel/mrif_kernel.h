// OriMRIFKernel -- host object of the MRI-FHD kernel
// (src/ori_kernel/mrif_kernel.{h,cu} of the reference).
#pragma once
#include "../Kernel.h"
#include "../header/mrif_header.h"

struct OriMRIFParamsStruct {
    int numK;
    int kGlobalIndex;
    float *x;
    float *y;
    float *z;
    float *outR;
    float *outI;
};

class OriMRIFKernel : public Kernel {
public:
    // numK = 2048 k-space samples, numX = 262144 voxels, seeded inputs; runs
    // ComputeRhoPhiGPU on the device and loads the k table into constant memory
    explicit OriMRIFKernel(int id);
    // caller-owned voxel arrays; the k table must already be loaded (setKValues)
    OriMRIFKernel(int id, int numK, const float *x, const float *y, const float *z, float *outR,
                  float *outI, int numX);
    ~OriMRIFKernel() override;

    void initParams() override;
    std::vector<int> getArgs() override { return std::vector<int>(); }
    OriMRIFParamsStruct *params() { return MRIFKernelParams; }
    int numX() const { return numX_; }
    // cudaMemcpyToSymbol(c, ...) of the reference (mrif_kernel.cu:304)
    static int setKValues(const mrif_kValues *kvals, int numK);

protected:
    void executeImpl(cudaStream_t stream) override;

private:
    void loadKernel() override {}
    void bind();
    OriMRIFParamsStruct *MRIFKernelParams = nullptr;
    int numX_ = 0;
};
