// OriCPKernel -- host object of the Coulomb-potential kernel
// (src/ori_kernel/cp_kernel.{h,cu} of the reference, float variant).
#pragma once
#include <string>

#include "../Kernel.h"
#include "../header/cp_header.h"

template <typename T>
struct OriCPParamsStruct {
    int numatoms;
    float gridspacing;
    T *energygrid;
};

// initatoms (cp_kernel.cu:185-209): glibc srand(54321) stream, 4 rand() per atom
void cpInitAtoms(float *atoms, int count, unsigned volx, unsigned voly, unsigned volz, float gridspacing);
// copyatomstoconstbuf (cp_kernel.cu:159-179): z -> (zplane - z)^2, then to constant memory
int cpCopyAtomsToConstBuf(const float *atoms, int count, float zplane);

class OriCPKernel : public Kernel {
public:
    // 4096 x 4096 slice at z = 0, spacing 0.1, atoms 1..64 of the 4000 generated
    explicit OriCPKernel(int id);
    OriCPKernel(int id, const std::string &moduleName, const std::string &kernelName);
    // caller-owned grid; atoms must already be loaded (cpCopyAtomsToConstBuf)
    OriCPKernel(int id, int numatoms, float gridspacing, float *energygrid, int volx, int voly);
    ~OriCPKernel() override;

    void initParams() override;   // callable again: re-zeroes the grid, reloads the atoms
    std::vector<int> getArgs() override { return std::vector<int>(); }
    OriCPParamsStruct<float> *params() { return CPKernelParams; }

protected:
    void executeImpl(cudaStream_t stream) override;

private:
    void loadKernel() override;
    OriCPParamsStruct<float> *CPKernelParams = nullptr;
    bool ownsGrid = false;
};
