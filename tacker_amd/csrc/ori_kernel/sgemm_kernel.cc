#include "sgemm_kernel.h"

#include <unordered_map>
#include <vector>

#include "../Logger.h"
#include "../rng.h"

extern Logger logger;
extern std::unordered_map<std::string, void *> fmap;

OriSGEMMKernel::OriSGEMMKernel(int id)
{
    Id = id;
    this->kernelName = "sgemm";
    initParams();
}

OriSGEMMKernel::OriSGEMMKernel(int id, const float *A, const float *B, float *C, int M, int N, int K)
{
    Id = id;
    this->kernelName = "sgemm";
    SGEMMKernelParams = new OriSGEMMParamsStruct{const_cast<float *>(A), const_cast<float *>(B), C, M, N, K};
    bind();
}

OriSGEMMKernel::~OriSGEMMKernel()
{
    if (holdsWorkspace) sgemmWorkspaceDone(SGEMMKernelParams->C);
    for (auto &ptr : cudaFreeList) tkErrCheck(tkFree(ptr));
    delete SGEMMKernelParams;
}

void OriSGEMMKernel::initParams()
{
    const int M = 4096, N = 4128, K = 4064;
    float *A = nullptr, *B = nullptr, *C = nullptr;
    auto dev = [&](float **p, size_t n) {
        TK_SAFE_CALL(tkMalloc((void **)p, n * sizeof(float)));
        cudaFreeList.push_back(*p);
    };
    dev(&A, (size_t)M * K);
    dev(&B, (size_t)K * N);
    dev(&C, (size_t)M * N);
    tk::Rng rng(1337ULL);
    std::vector<float> host((size_t)K * (M > N ? M : N));
    for (size_t i = 0; i < (size_t)M * K; ++i) host[i] = rng.uniform();
    TK_SAFE_CALL(tkMemcpy(A, host.data(), (size_t)M * K * sizeof(float), TK_MEMCPY_H2D));
    for (size_t i = 0; i < (size_t)K * N; ++i) host[i] = rng.uniform();
    TK_SAFE_CALL(tkMemcpy(B, host.data(), (size_t)K * N * sizeof(float), TK_MEMCPY_H2D));
    TK_SAFE_CALL(tkMemset(C, 0, (size_t)M * N * sizeof(float)));
    SGEMMKernelParams = new OriSGEMMParamsStruct{A, B, C, M, N, K};
    bind();
}

void OriSGEMMKernel::bind()
{
    OriSGEMMParamsStruct *p = SGEMMKernelParams;
    if (p->NORMAL_M <= 0 || p->NORMAL_N <= 0 || p->NORMAL_K <= 0 || p->NORMAL_M % SGEMM_TILE_M || p->NORMAL_N % SGEMM_TILE_N)
        logger.ERROR("sgemm: M must be a positive multiple of 128, N of 16, K positive");
    // Block positions: (x, y) = the reference's grid of 128 x 16 blocks of C
    // (src/ori_kernel/sgemm_kernel.cu:120-125), z = parts of SGEMM_K_CHUNK k steps.  The natural
    // launch below runs the (x, y) blocks, each through its whole k loop.
    const int parts = (p->NORMAL_K + SGEMM_K_CHUNK - 1) / SGEMM_K_CHUNK;
    launchGridDim = dim3(p->NORMAL_M / SGEMM_TILE_M, p->NORMAL_N / SGEMM_TILE_N, parts);
    launchBlockDim = dim3(SGEMM_TILE_N, SGEMM_TILE_TB_HEIGHT / 2, 1);   // one wavefront: a lane owns two of the block's rows
    kernelParams = {&p->A, &p->B, &p->C, &p->NORMAL_M, &p->NORMAL_N, &p->NORMAL_K};
    this->smem = 0;
    if (parts > 1 && !holdsWorkspace) {
        sgemmWorkspaceFor(p->C, p->NORMAL_M, p->NORMAL_N);
        holdsWorkspace = true;
    }
    auto it = fmap.find("ori_sgemm");
    this->kernelFunc = it == fmap.end() ? nullptr : it->second;
    this->initialized = true;
}

void OriSGEMMKernel::executeImpl(cudaStream_t stream)
{
    if (!kernelFunc) logger.ERROR("load kernel {ori_sgemm} failed!");
    const dim3 blocks(launchGridDim.x, launchGridDim.y, 1);
    TK_SAFE_CALL(tkLaunchKernel(this->kernelFunc, blocks.raw(), launchBlockDim.raw(),
                                (void **)this->kernelParams.data(), 0, stream));
}
