#include "cp_kernel.h"

#include <cstdlib>
#include <unordered_map>
#include <vector>

#include "../Logger.h"
#include "../ModuleCenter.h"

extern Logger logger;
extern ModuleCenter moduleCenter;
extern std::unordered_map<std::string, void *> fmap;

void cpInitAtoms(float *atoms, int count, unsigned volx, unsigned voly, unsigned volz, float gridspacing)
{
    // the box is held in unsigned ints, so 0.1f*4096 becomes 409 and 0.1f*1 becomes 0
    const unsigned sizex = (unsigned)(gridspacing * volx);
    const unsigned sizey = (unsigned)(gridspacing * voly);
    const unsigned sizez = (unsigned)(gridspacing * volz);
    srand(54321);
    for (int i = 0; i < count; i++) {
        float *a = atoms + 4 * i;
        a[0] = (rand() / (float)RAND_MAX) * sizex;
        a[1] = (rand() / (float)RAND_MAX) * sizey;
        a[2] = (rand() / (float)RAND_MAX) * sizez;
        a[3] = (float)(((rand() / (float)RAND_MAX) * 2.0) - 1.0);
    }
}

int cpCopyAtomsToConstBuf(const float *atoms, int count, float zplane)
{
    if (count > MAXATOMS) {
        printf("Atom count exceeds constant buffer storage capacity\n");
        return -1;
    }
    float atompre[4 * MAXATOMS];
    for (int i = 0; i < count * 4; i += 4) {
        atompre[i] = atoms[i];
        atompre[i + 1] = atoms[i + 1];
        const float dz = zplane - atoms[i + 2];
        atompre[i + 2] = dz * dz;
        atompre[i + 3] = atoms[i + 3];
    }
    return tkMemcpyToSymbol("atominfo", atompre, (size_t)count * 4 * sizeof(float), 0);
}

OriCPKernel::OriCPKernel(int id)
{
    Id = id;
    kernelName = "cp";
    moduleName = "ori_cp";
    initParams();
}

OriCPKernel::OriCPKernel(int id, const std::string &moduleName_, const std::string &kernelName_)
{
    Id = id;
    kernelName = kernelName_;
    moduleName = moduleName_;
    initParams();
}

OriCPKernel::OriCPKernel(int id, int numatoms, float gridspacing, float *energygrid, int volx, int voly)
{
    Id = id;
    kernelName = "cp";
    moduleName = "ori_cp";
    CPKernelParams = new OriCPParamsStruct<float>{numatoms, gridspacing, energygrid};
    launchBlockDim = dim3(BLOCKSIZEX, BLOCKSIZEY, 1);
    // z: the parts a block's unrolled x points are split into for the GPTB form's block
    // positions; the natural launch below runs the (x, y) blocks, each whole
    launchGridDim = dim3(volx / (BLOCKSIZEX * UNROLLX), voly / BLOCKSIZEY, CP_X_PARTS);
    kernelParams = {&CPKernelParams->numatoms, &CPKernelParams->gridspacing, &CPKernelParams->energygrid};
    auto it = fmap.find("ori_cp");
    kernelFunc = it == fmap.end() ? nullptr : it->second;
    smem = 0;
    initialized = true;
}

OriCPKernel::~OriCPKernel()
{
    if (ownsGrid && CPKernelParams) tkErrCheck(tkFree(CPKernelParams->energygrid));
    delete CPKernelParams;
    logger.DEBUG("id: " + std::to_string(Id) + " is destroyed!");
}

void OriCPKernel::initParams()
{
    std::vector<float> atoms((size_t)ATOMCOUNT * 4);
    const float gridspacing = 0.1f;
    const dim3 volsize(VOLSIZEX, VOLSIZEY, 1);
    cpInitAtoms(atoms.data(), ATOMCOUNT, volsize.x, volsize.y, volsize.z, gridspacing);
    const size_t volmemsz = sizeof(float) * volsize.x * volsize.y * volsize.z;

    float *output = nullptr;
    if (!this->initialized) {
        TK_SAFE_CALL(tkMalloc((void **)&output, volmemsz));
        TK_SAFE_CALL(tkMemset(output, 0, volmemsz));
        ownsGrid = true;
    } else {
        TK_SAFE_CALL(tkMemset(this->CPKernelParams->energygrid, 0, volmemsz));
    }
    const int atomstart = 1;
    const int runatoms = MAXATOMS;
    if (cpCopyAtomsToConstBuf(atoms.data() + 4 * atomstart, runatoms, 0 * gridspacing) != 0)
        logger.ERROR("cp: loading the atom table failed");

    if (!this->initialized) {
        CPKernelParams = new OriCPParamsStruct<float>{runatoms, 0.1f, output};
        launchBlockDim = dim3(BLOCKSIZEX, BLOCKSIZEY, 1);
        launchGridDim = dim3(volsize.x / (BLOCKSIZEX * UNROLLX), volsize.y / BLOCKSIZEY, CP_X_PARTS);
        kernelParams = {&CPKernelParams->numatoms, &CPKernelParams->gridspacing, &CPKernelParams->energygrid};
        auto it = fmap.find("ori_cp");
        kernelFunc = it == fmap.end() ? nullptr : it->second;
        smem = 0;
        initialized = true;
    }
}

void OriCPKernel::executeImpl(cudaStream_t stream)
{
    if (!kernelFunc) logger.ERROR("load kernel {ori_cp} failed!");
    const dim3 whole_blocks(launchGridDim.x, launchGridDim.y, 1);
    TK_SAFE_CALL(tkLaunchKernel(this->kernelFunc, whole_blocks.raw(), launchBlockDim.raw(),
                                (void **)this->kernelParams.data(), 0, stream));
}

// Optional path: take the function from a code object registered with the
// ModuleCenter instead of the built-in registry.
void OriCPKernel::loadKernel()
{
    logger.INFO("kernel name: " + kernelName + ", id: " + std::to_string(Id) + " is loading ...");
    this->function = moduleCenter.getFunction(moduleName, kernelName);
    if (this->function == nullptr)
        logger.ERROR("kernel name: " + kernelName + ", id: " + std::to_string(Id) + " load failed!");
}
