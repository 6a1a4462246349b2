// OriHOT3DKernel -- host object of Rodinia's hotspot3D step
// (src/ori_kernel/hot3d_kernel.{h,cu} of the reference).
#pragma once
#include "../Kernel.h"
#include "../header/hot3d_header.h"

struct OriHOT3DParamsStruct {
    float *p;
    float *tIn;
    float *tOut;
    float sdc;
    int nx;
    int ny;
    int nz;
    float ce, cw, cn, cs, ct, cb, cc;
};

// the step's coefficients for a chip of numCols x numRows x layers cells
// (src/ori_kernel/hot3d_kernel.cu:84-116: the same mixed float / double expressions)
void hot3dCoefficients(int numCols, int numRows, int layers, OriHOT3DParamsStruct *out);

class OriHOT3DKernel : public Kernel {
public:
    // 16384 x 8192 x 8 cells (src/ori_kernel/hot3d_kernel.cu:80-82).  The reference's temperature
    // and power arrays are all zero; here they are filled on the device, temperature uniform in
    // [320, 340) (seed 4101) and power in [0, 0.01) (seed 4102).
    explicit OriHOT3DKernel(int id);
    // caller-owned arrays of nx x ny x nz cells, coefficients as hot3dCoefficients gives them
    OriHOT3DKernel(int id, float *p, float *tIn, float *tOut, int nx, int ny, int nz);
    ~OriHOT3DKernel() override;

    void initParams() override;
    std::vector<int> getArgs() override { return std::vector<int>(); }
    OriHOT3DParamsStruct *params() { return HOT3DKernelParams; }

protected:
    void executeImpl(cudaStream_t stream) override;

private:
    void loadKernel() override {}
    void bind();
    OriHOT3DParamsStruct *HOT3DKernelParams = nullptr;
};
