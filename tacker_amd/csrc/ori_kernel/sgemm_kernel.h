// OriSGEMMKernel -- host object of Parboil's SGEMM kernel
// (src/ori_kernel/sgemm_kernel.{h,cu} of the reference).
#pragma once
#include "../Kernel.h"
#include "../header/sgemm_header.h"

struct OriSGEMMParamsStruct {
    float *A;
    float *B;
    float *C;
    int NORMAL_M;
    int NORMAL_N;
    int NORMAL_K;
};

// workspace of M x N floats bound to the output buffer C, where the partial results of a block
// rest between the k parts of the GPTB form; entered into the device table kernels look C up in
// (the one the GEMM role's shared reductions use, under a key of its own).  The caller is a user of
// the binding until sgemmWorkspaceDone(C); bindings without users go when room is needed.
void *sgemmWorkspaceFor(const float *C, int M, int N);
void sgemmWorkspaceDone(const float *C);

class OriSGEMMKernel : public Kernel {
public:
    // M, N, K = 4096, 4128, 4064, A and B uniform[0,1) from seed 1337, C zero
    // (src/ori_kernel/sgemm_kernel.cu:86-112)
    explicit OriSGEMMKernel(int id);
    // caller-owned matrices: A is K rows of M floats, B K rows of N floats, C N columns of M floats
    OriSGEMMKernel(int id, const float *A, const float *B, float *C, int M, int N, int K);
    ~OriSGEMMKernel() override;

    void initParams() override;
    std::vector<int> getArgs() override { return std::vector<int>(); }
    OriSGEMMParamsStruct *params() { return SGEMMKernelParams; }

protected:
    void executeImpl(cudaStream_t stream) override;

private:
    void loadKernel() override {}
    void bind();
    OriSGEMMParamsStruct *SGEMMKernelParams = nullptr;
    bool holdsWorkspace = false;
};
