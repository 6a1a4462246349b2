// OriMRIQKernel -- host object of the MRI-Q kernel
// (src/ori_kernel/mriq_kernel.{h,cu} of the reference).
#pragma once
#include "../Kernel.h"
#include "../header/mriq_header.h"

struct OriMRIQParamsStruct {
    int numK;
    int kGlobalIndex;
    float *x;
    float *y;
    float *z;
    float *Qr;
    float *Qi;
};

class OriMRIQKernel : public Kernel {
public:
    // numK = 2048 k-space samples, numX = 262144 voxels, seeded inputs; runs
    // ComputePhiMag on the device and loads the k table into constant memory
    explicit OriMRIQKernel(int id);
    // caller-owned voxel arrays; the k table must already be loaded (setKValues)
    OriMRIQKernel(int id, int numK, const float *x, const float *y, const float *z, float *Qr,
                  float *Qi, int numX);
    ~OriMRIQKernel() override;

    void initParams() override;
    std::vector<int> getArgs() override { return std::vector<int>(); }
    OriMRIQParamsStruct *params() { return MRIQKernelParams; }
    int numX() const { return numX_; }
    // cudaMemcpyToSymbol(ck, ...) of the reference (mriq_kernel.cu:254-256)
    static int setKValues(const mriq_kValues *kvals, int numK);

protected:
    void executeImpl(cudaStream_t stream) override;

private:
    void loadKernel() override {}
    void bind();
    OriMRIQParamsStruct *MRIQKernelParams = nullptr;
    int numX_ = 0;
};
