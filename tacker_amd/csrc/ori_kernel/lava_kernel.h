// OriLAVAKernel -- host object of Rodinia's lavaMD kernel
// (src/ori_kernel/lava_kernel.{h,cu} of the reference).
#pragma once
#include <vector>

#include "../Kernel.h"
#include "../header/lava_header.h"

struct OriLAVAParamsStruct {
    par_str d_par_gpu;
    dim_str d_dim_gpu;
    box_str *d_box_gpu;
    FOUR_VECTOR *d_rv_gpu;
    float *d_qv_gpu;
    FOUR_VECTOR *d_fv_gpu;
};

// the boxes of a boxes1d^3 system with their neighbour lists, x fastest
// (src/ori_kernel/lava_kernel.cu:176-224)
std::vector<box_str> lavaBoxes(int boxes1d);

class OriLAVAKernel : public Kernel {
public:
    // 60^3 boxes of 100 particles, alpha 0.5 (src/ori_kernel/lava_kernel.cu:163-175).  The
    // reference draws positions and charges from rand() seeded with the time of day; here they are
    // filled on the device, uniform in [0.1, 1) (seeds 4301, 4302), forces zero.
    explicit OriLAVAKernel(int id);
    // caller-owned particles: rv, fv = 100 boxes1d^3 {v, x, y, z}, qv as many charges; the box
    // list is built and kept by the object
    OriLAVAKernel(int id, float alpha, int boxes1d, FOUR_VECTOR *rv, float *qv, FOUR_VECTOR *fv);
    ~OriLAVAKernel() override;

    void initParams() override;
    std::vector<int> getArgs() override { return std::vector<int>(); }
    OriLAVAParamsStruct *params() { return LAVAKernelParams; }

protected:
    void executeImpl(cudaStream_t stream) override;

private:
    void loadKernel() override {}
    void bind(float alpha, int boxes1d, FOUR_VECTOR *rv, float *qv, FOUR_VECTOR *fv);
    OriLAVAParamsStruct *LAVAKernelParams = nullptr;
};
