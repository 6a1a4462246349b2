#include "cutcp_kernel.h"

#include <cmath>
#include <unordered_map>

#include "../Logger.h"
#include "../rng.h"

extern Logger logger;
extern std::unordered_map<std::string, void *> fmap;

bool cutcpPrepareInput(const float *atoms, int natoms, const float lo[3], int nx, int ny, int nz, float h, float cutoff,
                       CutcpBins *out, const char **why)
{
    static const char *none = "";
    if (why) *why = none;
    const int lnx = 8 * (int)ceilf(nx / 8.f), lny = 8 * (int)ceilf(ny / 8.f), lnz = 8 * (int)ceilf(nz / 8.f);
    const int c = (int)ceil(cutoff * BIN_INVLEN);   // padding bins around the lattice
    out->padding = c;
    out->binDim[0] = (int)ceil(lnx * h * BIN_INVLEN) + 2 * c;
    out->binDim[1] = (int)ceil(lny * h * BIN_INVLEN) + 2 * c;
    out->binDim[2] = (int)ceil(lnz * h * BIN_INVLEN) + 2 * c;
    const long long nbins = (long long)out->binDim[0] * out->binDim[1] * out->binDim[2];

    // neighbour list: every bin offset whose bin can hold an atom within the cutoff of a point of a
    // region centred on one bin (regions no wider than a bin) or on a cube of 3 x 3 x 3 bins
    float s;
    int needs;
    if (ceilf(BIN_LENGTH / (8 * h)) == floorf(BIN_LENGTH / (8 * h))) {
        s = sqrtf(3);
        needs = 2 * c + 1;
    } else if (8 * h <= 2 * BIN_LENGTH) {
        s = 2.f * sqrtf(3);
        needs = 2 * c + 3;
    } else {
        if (why) *why = "cutcp: the lattice spacing must be at most a quarter of the bin length";
        return false;
    }
    if (needs > NBRLIST_DIM) {
        if (why) *why = "cutcp: the cutoff reaches past the neighbour list";
        return false;
    }
    const float r2 = (cutoff + s * BIN_LENGTH) * (cutoff + s * BIN_LENGTH);
    out->nbrlist.clear();
    for (int k = -c; k <= c; k++)
        for (int j = -c; j <= c; j++)
            for (int i = -c; i <= c; i++) {
                if ((i * i + j * j + k * k) * BIN_LENGTH * BIN_LENGTH >= r2) continue;
                out->nbrlist.push_back(i);
                out->nbrlist.push_back(j);
                out->nbrlist.push_back(k);
            }

    // geometric hashing of the atoms into the bins, in the order given
    out->bins.assign((size_t)nbins * BIN_SIZE, 0.0f);
    std::vector<int> count((size_t)nbins, 0);
    out->extra = out->excluded = 0;
    for (int n = 0; n < natoms; n++) {
        const float px = atoms[4 * n] - lo[0], py = atoms[4 * n + 1] - lo[1], pz = atoms[4 * n + 2] - lo[2];
        const float q = atoms[4 * n + 3];
        const int i = (int)floorf(px * BIN_INVLEN), j = (int)floorf(py * BIN_INVLEN), k = (int)floorf(pz * BIN_INVLEN);
        if (i >= -c && i < out->binDim[0] - c && j >= -c && j < out->binDim[1] - c && k >= -c && k < out->binDim[2] - c &&
            q != 0) {
            const long long index = ((long long)(k + c) * out->binDim[1] + (j + c)) * out->binDim[0] + (i + c);
            if (count[index] < BIN_DEPTH) {
                float *slot = out->bins.data() + index * BIN_SIZE + 4 * count[index];
                slot[0] = px, slot[1] = py, slot[2] = pz, slot[3] = q;
                count[index]++;
            } else {
                out->extra++;
            }
        } else {
            out->excluded++;
        }
    }
    return true;
}

static int g_neighbour_len = 0;   // what the device table holds

int cutcpSetNeighbours(const int *ijk, int len)
{
    if (len < 0 || len > NBRLIST_MAXLEN) return TK_ERROR_INVALID_VALUE;
    int rc = tkMemcpyToSymbol("NbrListLen", &len, sizeof(int), 0);
    if (!rc && len) rc = tkMemcpyToSymbol("NbrList", ijk, (size_t)len * 3 * sizeof(int), 0);
    if (!rc) g_neighbour_len = len;
    return rc;
}

int cutcpNeighbourParts()
{
    const int parts = (g_neighbour_len + CUTCP_NBR_CHUNK - 1) / CUTCP_NBR_CHUNK;
    return parts < 1 ? 1 : parts;
}

OriCUTCPKernel::OriCUTCPKernel(int id)
{
    Id = id;
    this->kernelName = "cutcp";
    initParams();
}

OriCUTCPKernel::OriCUTCPKernel(int id, int binDim_x, int binDim_y, float *binZeroAddr, float h, float cutoff2,
                               float inv_cutoff2, float *regionZeroAddr, int rx, int ry, int rz)
{
    Id = id;
    this->kernelName = "cutcp";
    CUTCPKernelParams = new OriCUTCPParamsStruct{binDim_x, binDim_y, binZeroAddr, h, cutoff2, inv_cutoff2, regionZeroAddr, 0};
    bind(rx, ry, rz);
}

OriCUTCPKernel::~OriCUTCPKernel()
{
    for (auto &ptr : cudaFreeList) tkErrCheck(tkFree(ptr));
    delete CUTCPKernelParams;
}

void OriCUTCPKernel::initParams()
{
    const float h = 0.5f, cutoff = 12.f;
    const int n = 208;                       // lattice points per dimension: 26 regions
    const float box = (n - 1) * h;           // atoms fill the lattice's box
    const int natoms = 70000;                // about 4 per bin: few bins overflow their 8 slots
    std::vector<float> atoms((size_t)natoms * 4);
    tk::Rng rng(54321ULL);
    for (int i = 0; i < natoms; ++i) {
        atoms[4 * i] = rng.uniform() * box;
        atoms[4 * i + 1] = rng.uniform() * box;
        atoms[4 * i + 2] = rng.uniform() * box;
        atoms[4 * i + 3] = rng.uniform() * 2.0f - 1.0f;
    }
    const float lo[3] = {0.f, 0.f, 0.f};
    CutcpBins bins;
    const char *why = nullptr;
    if (!cutcpPrepareInput(atoms.data(), natoms, lo, n, n, n, h, cutoff, &bins, &why)) logger.ERROR(why);
    if (cutcpSetNeighbours(bins.nbrlist.data(), (int)bins.nbrlist.size() / 3) != 0)
        logger.ERROR("cutcp: loading the neighbour list failed");

    float *binBase = nullptr, *regions = nullptr;
    const size_t lnall = (size_t)n * n * n;
    TK_SAFE_CALL(tkMalloc((void **)&binBase, bins.bins.size() * sizeof(float)));
    cudaFreeList.push_back(binBase);
    TK_SAFE_CALL(tkMemcpy(binBase, bins.bins.data(), bins.bins.size() * sizeof(float), TK_MEMCPY_H2D));
    TK_SAFE_CALL(tkMalloc((void **)&regions, lnall * sizeof(float)));
    cudaFreeList.push_back(regions);
    TK_SAFE_CALL(tkMemset(regions, 0, lnall * sizeof(float)));
    // cutoff2 and inv_cutoff2 as the reference types them (src/ori_kernel/cutcp_kernel.cu:226-227)
    CUTCPKernelParams = new OriCUTCPParamsStruct{bins.binDim[0], bins.binDim[1], binBase + bins.zeroOffsetFloats(), h,
                                                 144.0f, 0.006944f, regions, 25};
    bind(n / 8, n / 8, 2);   // grid.z = 2: the two lowest layers of regions (:249)
}

void OriCUTCPKernel::bind(int rx, int ry, int rz)
{
    if (rx <= 0 || ry <= 0 || rz <= 0) logger.ERROR("cutcp: the grid of regions must not be empty");
    OriCUTCPParamsStruct *p = CUTCPKernelParams;
    // Block positions: (x, y, z / parts) = the reference's grid of regions
    // (src/ori_kernel/cutcp_kernel.cu:246-249), the parts of the neighbour list folded into z as the
    // slowest index.  The natural launch below runs the regions, each through the whole list.
    regionsZ = rz;
    launchGridDim = dim3(rx, ry, rz * cutcpNeighbourParts());
    launchBlockDim = dim3(8, 2, 8);
    kernelParams = {&p->binDim_x, &p->binDim_y, &p->binZeroAddr, &p->h, &p->cutoff2, &p->inv_cutoff2, &p->regionZeroAddr,
                    &p->zRegionIndex_t};
    this->smem = 0;
    auto it = fmap.find("ori_cutcp");
    this->kernelFunc = it == fmap.end() ? nullptr : it->second;
    this->initialized = true;
}

void OriCUTCPKernel::executeImpl(cudaStream_t stream)
{
    if (!kernelFunc) logger.ERROR("load kernel {ori_cutcp} failed!");
    const dim3 regions(launchGridDim.x, launchGridDim.y, regionsZ);
    TK_SAFE_CALL(tkLaunchKernel(this->kernelFunc, regions.raw(), launchBlockDim.raw(),
                                (void **)this->kernelParams.data(), 0, stream));
}
