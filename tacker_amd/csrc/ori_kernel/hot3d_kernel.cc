#include "hot3d_kernel.h"

#include <unordered_map>

#include "../Logger.h"
#include "fill.h"

extern Logger logger;
extern std::unordered_map<std::string, void *> fmap;

void hot3dCoefficients(int numCols, int numRows, int layers, OriHOT3DParamsStruct *out)
{
    // cell size, thermal capacitance and resistances of a cell, and the largest stable step
    const float t_chip = HOT3D_T_CHIP, chip_height = HOT3D_CHIP_HEIGHT, chip_width = HOT3D_CHIP_WIDTH;
    const float dx = chip_height / numRows;
    const float dy = chip_width / numCols;
    const float dz = t_chip / layers;
    const float Cap = HOT3D_FACTOR_CHIP * HOT3D_SPEC_HEAT_SI * t_chip * dx * dy;
    const float Rx = dy / (2.0 * HOT3D_K_SI * t_chip * dx);
    const float Ry = dx / (2.0 * HOT3D_K_SI * t_chip * dy);
    const float Rz = dz / (HOT3D_K_SI * dx * dy);
    const float max_slope = HOT3D_MAX_PD / (HOT3D_FACTOR_CHIP * t_chip * HOT3D_SPEC_HEAT_SI);
    const float dt = HOT3D_PRECISION / max_slope;
    const float stepDivCap = dt / Cap;
    out->sdc = stepDivCap;
    out->ce = out->cw = stepDivCap / Rx;
    out->cn = out->cs = stepDivCap / Ry;
    out->ct = out->cb = stepDivCap / Rz;
    out->cc = 1.0 - (2.0 * out->ce + 2.0 * out->cn + 3.0 * out->ct);
}

OriHOT3DKernel::OriHOT3DKernel(int id)
{
    Id = id;
    this->kernelName = "hot3d";
    initParams();
}

OriHOT3DKernel::OriHOT3DKernel(int id, float *p, float *tIn, float *tOut, int nx, int ny, int nz)
{
    Id = id;
    this->kernelName = "hot3d";
    HOT3DKernelParams = new OriHOT3DParamsStruct{};
    HOT3DKernelParams->p = p;
    HOT3DKernelParams->tIn = tIn;
    HOT3DKernelParams->tOut = tOut;
    HOT3DKernelParams->nx = nx;
    HOT3DKernelParams->ny = ny;
    HOT3DKernelParams->nz = nz;
    bind();
}

OriHOT3DKernel::~OriHOT3DKernel()
{
    for (auto &ptr : cudaFreeList) tkErrCheck(tkFree(ptr));
    delete HOT3DKernelParams;
}

void OriHOT3DKernel::initParams()
{
    const int numCols = 1024 * 8 * 2, numRows = 1024 * 8, layers = 8;
    const size_t cells = (size_t)numCols * numRows * layers;
    float *arrays[3] = {nullptr, nullptr, nullptr};   // power, temperature in, temperature out
    for (auto &a : arrays) {
        TK_SAFE_CALL(tkMalloc((void **)&a, cells * sizeof(float)));
        cudaFreeList.push_back(a);
    }
    tkFillUniform(arrays[0], cells, 4102u, 0.0f, 0.01f);
    tkFillUniform(arrays[1], cells, 4101u, 320.0f, 340.0f);
    TK_SAFE_CALL(tkMemset(arrays[2], 0, cells * sizeof(float)));
    HOT3DKernelParams = new OriHOT3DParamsStruct{};
    HOT3DKernelParams->p = arrays[0];
    HOT3DKernelParams->tIn = arrays[1];
    HOT3DKernelParams->tOut = arrays[2];
    HOT3DKernelParams->nx = numCols;
    HOT3DKernelParams->ny = numRows;
    HOT3DKernelParams->nz = layers;
    bind();
}

void OriHOT3DKernel::bind()
{
    OriHOT3DParamsStruct *q = HOT3DKernelParams;
    if (q->nx < HOT3D_TILE_X || q->nx % HOT3D_TILE_X || q->ny < HOT3D_TILE_Y || q->ny % HOT3D_TILE_Y || q->nz < 2)
        logger.ERROR("hot3d: nx a multiple of 64, ny a multiple of 4, at least two layers (the reference's launch "
                     "has no partial blocks and reads the second layer unconditionally)");
    hot3dCoefficients(q->nx, q->ny, q->nz, q);
    launchGridDim = dim3(q->nx / HOT3D_TILE_X, q->ny / HOT3D_TILE_Y, 1);
    launchBlockDim = dim3(HOT3D_TILE_X, HOT3D_TILE_Y, 1);
    kernelParams = {&q->p,  &q->tIn, &q->tOut, &q->sdc, &q->nx, &q->ny, &q->nz,
                    &q->ce, &q->cw,  &q->cn,   &q->cs,  &q->ct, &q->cb, &q->cc};
    this->smem = 0;
    auto it = fmap.find("ori_hot3d");
    this->kernelFunc = it == fmap.end() ? nullptr : it->second;
    this->initialized = true;
}

void OriHOT3DKernel::executeImpl(cudaStream_t stream)
{
    if (!kernelFunc) logger.ERROR("load kernel {ori_hot3d} failed!");
    TK_SAFE_CALL(tkLaunchKernel(this->kernelFunc, launchGridDim.raw(), launchBlockDim.raw(),
                                (void **)this->kernelParams.data(), 0, stream));
}
