#include "mrif_kernel.h"

#include <unordered_map>
#include <vector>

#include "../Logger.h"
#include "../rng.h"

extern Logger logger;
extern std::unordered_map<std::string, void *> fmap;

OriMRIFKernel::OriMRIFKernel(int id)
{
    Id = id;
    this->kernelName = "mrif";
    initParams();
}

OriMRIFKernel::OriMRIFKernel(int id, int numK, const float *x, const float *y, const float *z,
                             float *outR, float *outI, int numX)
    : numX_(numX)
{
    Id = id;
    this->kernelName = "mrif";
    MRIFKernelParams = new OriMRIFParamsStruct{numK, 0, const_cast<float *>(x), const_cast<float *>(y),
                                               const_cast<float *>(z), outR, outI};
    bind();
}

OriMRIFKernel::~OriMRIFKernel()
{
    for (auto &ptr : cudaFreeList) tkErrCheck(tkFree(ptr));
    delete MRIFKernelParams;
}

int OriMRIFKernel::setKValues(const mrif_kValues *kvals, int numK)
{
    if (numK < 0 || numK > MRIF_MAX_K) return TK_ERROR_INVALID_VALUE;
    return tkMemcpyToSymbol("c_mrif", kvals, (size_t)numK * sizeof(mrif_kValues), 0);
}

// The reference reads an input file that is not shipped and uses the first 256
// samples of its table (src/ori_kernel/mrif_kernel.cu:31,84-85,298-304).  Here:
// numK = 2048, numX = 262144, kx,ky,kz and voxel coordinates uniform[-0.5,0.5),
// phi and d uniform[0,1), out = 0, same flow (device ComputeRhoPhiGPU -> host AoS
// table -> constant memory).
void OriMRIFKernel::initParams()
{
    const int numK = 2048;
    numX_ = 262144;
    tk::Rng rng(1337ULL);
    std::vector<float> kx(numK), ky(numK), kz(numK), phiR(numK), phiI(numK), dR(numK), dI(numK);
    std::vector<float> x(numX_), y(numX_), z(numX_);
    for (int k = 0; k < numK; ++k) kx[k] = rng.uniform(-0.5f, 0.5f);
    for (int k = 0; k < numK; ++k) ky[k] = rng.uniform(-0.5f, 0.5f);
    for (int k = 0; k < numK; ++k) kz[k] = rng.uniform(-0.5f, 0.5f);
    for (int i = 0; i < numX_; ++i) x[i] = rng.uniform(-0.5f, 0.5f);
    for (int i = 0; i < numX_; ++i) y[i] = rng.uniform(-0.5f, 0.5f);
    for (int i = 0; i < numX_; ++i) z[i] = rng.uniform(-0.5f, 0.5f);
    for (int k = 0; k < numK; ++k) phiR[k] = rng.uniform();
    for (int k = 0; k < numK; ++k) phiI[k] = rng.uniform();
    for (int k = 0; k < numK; ++k) dR[k] = rng.uniform();
    for (int k = 0; k < numK; ++k) dI[k] = rng.uniform();

    float *d_phiR, *d_phiI, *d_dR, *d_dI, *d_rRhoPhi, *d_iRhoPhi, *d_x, *d_y, *d_z, *d_outR, *d_outI;
    auto dev = [&](float **p, size_t n) {
        TK_SAFE_CALL(tkMalloc((void **)p, n * sizeof(float)));
        cudaFreeList.push_back(*p);
    };
    dev(&d_phiR, numK); dev(&d_phiI, numK); dev(&d_dR, numK); dev(&d_dI, numK);
    dev(&d_rRhoPhi, numK); dev(&d_iRhoPhi, numK);
    dev(&d_x, numX_); dev(&d_y, numX_); dev(&d_z, numX_); dev(&d_outR, numX_); dev(&d_outI, numX_);
    TK_SAFE_CALL(tkMemcpy(d_phiR, phiR.data(), numK * sizeof(float), TK_MEMCPY_H2D));
    TK_SAFE_CALL(tkMemcpy(d_phiI, phiI.data(), numK * sizeof(float), TK_MEMCPY_H2D));
    TK_SAFE_CALL(tkMemcpy(d_dR, dR.data(), numK * sizeof(float), TK_MEMCPY_H2D));
    TK_SAFE_CALL(tkMemcpy(d_dI, dI.data(), numK * sizeof(float), TK_MEMCPY_H2D));
    TK_SAFE_CALL(tkMemcpy(d_x, x.data(), numX_ * sizeof(float), TK_MEMCPY_H2D));
    TK_SAFE_CALL(tkMemcpy(d_y, y.data(), numX_ * sizeof(float), TK_MEMCPY_H2D));
    TK_SAFE_CALL(tkMemcpy(d_z, z.data(), numX_ * sizeof(float), TK_MEMCPY_H2D));
    TK_SAFE_CALL(tkMemset(d_outR, 0, numX_ * sizeof(float)));
    TK_SAFE_CALL(tkMemset(d_outI, 0, numX_ * sizeof(float)));

    // RhoPhi on the device (ComputeRhoPhiGPU), then back for the AoS table
    auto it = fmap.find("ComputeRhoPhiGPU");
    if (it == fmap.end()) logger.ERROR("load kernel {ComputeRhoPhiGPU} failed!");
    int nk = numK;
    void *args[] = {&nk, &d_phiR, &d_phiI, &d_dR, &d_dI, &d_rRhoPhi, &d_iRhoPhi};
    const dim3 grid((numK + KERNEL_RHO_PHI_THREADS_PER_BLOCK - 1) / KERNEL_RHO_PHI_THREADS_PER_BLOCK);
    TK_SAFE_CALL(tkLaunchKernel(it->second, grid.raw(), dim3(KERNEL_RHO_PHI_THREADS_PER_BLOCK).raw(),
                                args, 0, nullptr));
    std::vector<float> rRhoPhi(numK), iRhoPhi(numK);
    TK_SAFE_CALL(tkMemcpy(rRhoPhi.data(), d_rRhoPhi, numK * sizeof(float), TK_MEMCPY_D2H));
    TK_SAFE_CALL(tkMemcpy(iRhoPhi.data(), d_iRhoPhi, numK * sizeof(float), TK_MEMCPY_D2H));
    std::vector<mrif_kValues> kVals(numK);
    for (int k = 0; k < numK; ++k) kVals[k] = mrif_kValues{kx[k], ky[k], kz[k], rRhoPhi[k], iRhoPhi[k]};
    TK_SAFE_CALL(setKValues(kVals.data(), numK));

    MRIFKernelParams = new OriMRIFParamsStruct{numK, 0, d_x, d_y, d_z, d_outR, d_outI};
    bind();
}

void OriMRIFKernel::bind()
{
    if (numX_ % KERNEL_FH_THREADS_PER_BLOCK != 0)
        logger.ERROR("mrif: numX must be a multiple of 256");
    OriMRIFParamsStruct *p = MRIFKernelParams;
    // Block positions: x = blocks of 256 voxels, y = chunks of MRIF_K_CHUNK k records (the
    // reference's loop over grids of the k table, mrif_kernel.cu:84-85, as a grid dimension).
    // The natural launch below runs one workgroup per voxel block, which walks all chunks.
    const int chunks = p->numK > 0 ? (p->numK + MRIF_K_CHUNK - 1) / MRIF_K_CHUNK : 1;
    launchGridDim = dim3(numX_ / KERNEL_FH_THREADS_PER_BLOCK, chunks, 1);
    launchBlockDim = dim3(KERNEL_FH_THREADS_PER_BLOCK, 1, 1);
    kernelParams = {&p->numK, &p->kGlobalIndex, &p->x, &p->y, &p->z, &p->outR, &p->outI};
    this->smem = 0;
    auto it = fmap.find("ori_mrif");
    this->kernelFunc = it == fmap.end() ? nullptr : it->second;
    this->initialized = true;
}

void OriMRIFKernel::executeImpl(cudaStream_t stream)
{
    if (!kernelFunc) logger.ERROR("load kernel {ori_mrif} failed!");
    const dim3 voxel_blocks(launchGridDim.x, 1, 1);
    TK_SAFE_CALL(tkLaunchKernel(this->kernelFunc, voxel_blocks.raw(), launchBlockDim.raw(),
                                (void **)this->kernelParams.data(), 0, stream));
}
