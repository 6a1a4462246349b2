// OriPATHKernel -- host object of Rodinia's pathfinder step
// (src/ori_kernel/path_kernel.{h,cu} of the reference).
#pragma once
#include "../Kernel.h"
#include "../header/path_header.h"

struct OriPATHParamsStruct {
    int iteration;
    int *gpuWall;
    int *gpuSrc;
    int *gpuResults;
    int cols;
    int rows;
    int startStep;
    int border;
};

// block positions of a launch over `cols` columns with a pyramid of `iteration` rows
// (src/ori_kernel/path_kernel.cu:121-123)
int pathBlocks(int cols, int iteration);

class OriPATHKernel : public Kernel {
public:
    // 1000000 x 1200 cells of rand() % 10 after srand(9), pyramid height 125
    // (src/ori_kernel/path_kernel.cu:102-120): the first row is the source, the rest the wall.  One
    // launch reads the wall's first 125 rows; those and the source come from the same rand()
    // sequence as the reference's, the rows below them are filled on the device (seed 4201).
    explicit OriPATHKernel(int id);
    // caller-owned arrays: the wall without its first row, source and result rows of `cols` values
    OriPATHKernel(int id, int iteration, int *gpuWall, int *gpuSrc, int *gpuResults, int cols, int rows, int startStep);
    ~OriPATHKernel() override;

    void initParams() override;
    std::vector<int> getArgs() override { return std::vector<int>(); }
    OriPATHParamsStruct *params() { return PATHKernelParams; }

protected:
    void executeImpl(cudaStream_t stream) override;

private:
    void loadKernel() override {}
    void bind();
    OriPATHParamsStruct *PATHKernelParams = nullptr;
};
