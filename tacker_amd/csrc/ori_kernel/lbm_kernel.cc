#include "lbm_kernel.h"

#include <cstring>
#include <unordered_map>
#include <vector>

#include "../Logger.h"
#include "../header/lbm_header.h"
#include "../rng.h"

extern Logger logger;
extern std::unordered_map<std::string, void *> fmap;

OriLBMKernel::OriLBMKernel(int id)
{
    Id = id;
    this->kernelName = "lbm";
    initParams();
}

OriLBMKernel::OriLBMKernel(int id, const float *src, float *dst, int sx, int sy, int sz)
    : sx_(sx), sy_(sy), sz_(sz)
{
    Id = id;
    this->kernelName = "lbm";
    LBMKernelParams = new OriLBMParamsStruct{const_cast<float *>(src), dst};
    bind();
}

OriLBMKernel::~OriLBMKernel()
{
    for (auto &ptr : cudaFreeList) tkErrCheck(tkFree(ptr));
    delete LBMKernelParams;
}

// Benchmark lattice: 120 x 120 x 150 cells.  Allocation = cells*20 floats plus
// TOTAL_MARGIN floats at each end, kernel pointers advanced by REAL_MARGIN
// (src/ori_kernel/lbm_kernel.cu:190,215-216, src/header/lbm_header.h:244-245).
// Contents: the 19 distributions are the rest equilibrium w_i plus uniform
// [0,1e-3) noise (keeps rho > 0); FLAGS has OBSTACLE on ~5% of the cells and
// ACCEL nowhere.  (The reference fills every plane, FLAGS included, with cuRAND
// floats, which makes half the cells obstacles by accident of mantissa bits.)
void OriLBMKernel::initParams()
{
    sx_ = 120;
    sy_ = 120;
    sz_ = 150;
    const size_t cells = (size_t)sx_ * sy_ * sz_;
    const size_t margin = (size_t)LBM_TOTAL_MARGIN(sx_, sy_);
    const size_t floats = cells * LBM_N_CELL_ENTRIES + 2 * margin;

    static const float w[19] = {LBM_DFL1, LBM_DFL2, LBM_DFL2, LBM_DFL2, LBM_DFL2, LBM_DFL2, LBM_DFL2,
                                LBM_DFL3, LBM_DFL3, LBM_DFL3, LBM_DFL3, LBM_DFL3, LBM_DFL3, LBM_DFL3,
                                LBM_DFL3, LBM_DFL3, LBM_DFL3, LBM_DFL3, LBM_DFL3};
    std::vector<float> host(floats, 0.0f);
    float *grid = host.data() + LBM_REAL_MARGIN(sx_, sy_);
    tk::Rng rng(1337ULL);
    for (int e = 0; e < 19; ++e)
        for (size_t c = 0; c < cells; ++c) grid[cells * e + c] = w[e] + 1e-3f * rng.uniform();
    for (size_t c = 0; c < cells; ++c) {
        const unsigned flag = rng.uniform() < 0.05f ? (unsigned)LBM_OBSTACLE : 0u;
        std::memcpy(&grid[cells * LBM_FLAGS + c], &flag, 4);
    }

    float *src = nullptr, *dst = nullptr;
    TK_SAFE_CALL(tkMalloc((void **)&src, floats * sizeof(float)));
    TK_SAFE_CALL(tkMalloc((void **)&dst, floats * sizeof(float)));
    cudaFreeList.push_back(src);
    cudaFreeList.push_back(dst);
    TK_SAFE_CALL(tkMemcpy(src, host.data(), floats * sizeof(float), TK_MEMCPY_H2D));
    TK_SAFE_CALL(tkMemcpy(dst, src, floats * sizeof(float), TK_MEMCPY_D2D));

    LBMKernelParams = new OriLBMParamsStruct{src + LBM_REAL_MARGIN(sx_, sy_), dst + LBM_REAL_MARGIN(sx_, sy_)};
    bind();
}

void OriLBMKernel::bind()
{
    if ((long long)sx_ * sy_ * sz_ * LBM_N_CELL_ENTRIES >= (1LL << 31))
        logger.ERROR("lbm: grid too large for 32-bit cell indices");
    launchBlockDim = dim3(sx_, 1, 1);
    launchGridDim = dim3(sy_, sz_, 1);
    kernelParams = {&LBMKernelParams->src, &LBMKernelParams->dst};
    this->smem = 0;
    auto it = fmap.find("ori_lbm");
    this->kernelFunc = it == fmap.end() ? nullptr : it->second;
    this->initialized = true;
}

void OriLBMKernel::swapGrids()
{
    float *t = LBMKernelParams->src;
    LBMKernelParams->src = LBMKernelParams->dst;
    LBMKernelParams->dst = t;
}

void OriLBMKernel::executeImpl(cudaStream_t stream)
{
    if (!kernelFunc) logger.ERROR("load kernel {ori_lbm} failed!");
    if (sx_ > 1024) logger.ERROR("ori_lbm: SIZE_X above 1024 needs the GPTB form");
    TK_SAFE_CALL(tkLaunchKernel(this->kernelFunc, launchGridDim.raw(), launchBlockDim.raw(),
                                (void **)this->kernelParams.data(), 0, stream));
}
