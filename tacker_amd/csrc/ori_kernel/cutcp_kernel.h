// OriCUTCPKernel -- host object of Parboil's cutoff Coulomb potential
// (src/ori_kernel/cutcp_kernel.{h,cu}, src/header/cutcp_header.h of the reference).
#pragma once
#include <vector>

#include "../Kernel.h"
#include "../header/cutcp_header.h"

struct OriCUTCPParamsStruct {
    int binDim_x;
    int binDim_y;
    float *binZeroAddr;      // bin (0, 0, 0) of the lattice, behind the padding bins
    float h;
    float cutoff2;
    float inv_cutoff2;
    float *regionZeroAddr;   // energies, region after region, 512 floats each
    int zRegionIndex_t;      // carried, never read (as in the reference)
};

// What prepare_input (src/header/cutcp_header.h:111-300) builds from a list of atoms: the atoms hashed
// into bins of 4 x 4 x 4 Angstroms, BIN_DEPTH to a bin with c padding bins on every side, and the
// list of bin offsets a region has to visit.
struct CutcpBins {
    int binDim[3] = {0, 0, 0};
    int padding = 0;                  // c: padding bins per side
    std::vector<float> bins;          // binDim x*y*z bins of BIN_DEPTH {x, y, z, q}, x fastest
    std::vector<int> nbrlist;         // (i, j, k) triples
    int extra = 0;                    // atoms that found their bin full (the reference leaves them to the CPU)
    int excluded = 0;                 // atoms outside the bins or without charge
    long long zeroOffsetFloats() const
    {
        return (((long long)padding * binDim[1] + padding) * binDim[0] + padding) * BIN_SIZE;
    }
};
// atoms: natoms x {x, y, z, q}; lo: lowest corner of the lattice; nx, ny, nz lattice points with spacing h.
// Returns false (and says why in *why) where the reference's function returns -1.
bool cutcpPrepareInput(const float *atoms, int natoms, const float lo[3], int nx, int ny, int nz, float h, float cutoff,
                       CutcpBins *out, const char **why);
// cudaMemcpyToSymbol(NbrListLen / NbrList) (src/ori_kernel/cutcp_kernel.cu:241-242)
int cutcpSetNeighbours(const int *ijk, int len);
// parts of CUTCP_NBR_CHUNK entries the neighbour list loaded last falls into (1 for an empty list):
// the rows of the GPTB position grid of kernel objects built from now on
int cutcpNeighbourParts();

class OriCUTCPKernel : public Kernel {
public:
    // a lattice of 208^3 points, spacing 0.5, cutoff 12; grid (26, 26, 2): the two lowest layers of
    // regions (src/ori_kernel/cutcp_kernel.cu:181-263).  The reference reads its atoms from a file it
    // does not ship; here 70000 atoms with seeded uniform positions in the box and charges in [-1, 1).
    explicit OriCUTCPKernel(int id);
    // caller-owned bins and energies; the neighbour list must have been loaded (cutcpSetNeighbours)
    // and must not change its number of parts while the object is in use
    OriCUTCPKernel(int id, int binDim_x, int binDim_y, float *binZeroAddr, float h, float cutoff2, float inv_cutoff2,
                   float *regionZeroAddr, int regions_x, int regions_y, int regions_z);
    ~OriCUTCPKernel() override;

    void initParams() override;
    std::vector<int> getArgs() override { return std::vector<int>(); }
    OriCUTCPParamsStruct *params() { return CUTCPKernelParams; }

protected:
    void executeImpl(cudaStream_t stream) override;

private:
    void loadKernel() override {}
    void bind(int rx, int ry, int rz);
    OriCUTCPParamsStruct *CUTCPKernelParams = nullptr;
    int regionsZ = 0;   // launchGridDim.z also counts the parts of the neighbour list
};
