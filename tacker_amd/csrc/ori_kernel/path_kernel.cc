#include "path_kernel.h"

#include <cstdlib>
#include <unordered_map>
#include <vector>

#include "../Logger.h"
#include "fill.h"

extern Logger logger;
extern std::unordered_map<std::string, void *> fmap;

int pathBlocks(int cols, int iteration)
{
    const int small = PATH_BLOCK_SIZE - iteration * PATH_HALO * 2;
    if (small <= 0 || cols <= 0) return 0;
    return cols / small + (cols % small == 0 ? 0 : 1);
}

OriPATHKernel::OriPATHKernel(int id)
{
    Id = id;
    this->kernelName = "path";
    initParams();
}

OriPATHKernel::OriPATHKernel(int id, int iteration, int *gpuWall, int *gpuSrc, int *gpuResults, int cols, int rows,
                             int startStep)
{
    Id = id;
    this->kernelName = "path";
    PATHKernelParams =
        new OriPATHParamsStruct{iteration, gpuWall, gpuSrc, gpuResults, cols, rows, startStep, iteration * PATH_HALO};
    bind();
}

OriPATHKernel::~OriPATHKernel()
{
    for (auto &ptr : cudaFreeList) tkErrCheck(tkFree(ptr));
    delete PATHKernelParams;
}

void OriPATHKernel::initParams()
{
    const int rows = 1000000, cols = 1200, pyramid_height = 125;
    const size_t wall_cells = (size_t)(rows - 1) * cols;
    int *wall = nullptr, *result[2] = {nullptr, nullptr};
    TK_SAFE_CALL(tkMalloc((void **)&result[0], sizeof(int) * cols));
    TK_SAFE_CALL(tkMalloc((void **)&result[1], sizeof(int) * cols));
    TK_SAFE_CALL(tkMalloc((void **)&wall, sizeof(int) * wall_cells));
    cudaFreeList.push_back(result[0]);
    cudaFreeList.push_back(result[1]);
    cudaFreeList.push_back(wall);
    // rows 0 .. pyramid_height in the reference's order; row 0 is the source
    std::vector<int> head((size_t)(pyramid_height + 1) * cols);
    srand(PATH_SEED);
    for (auto &v : head) v = rand() % 10;
    tkFillIntMod(wall, wall_cells, 4201u, 10);
    TK_SAFE_CALL(tkMemcpy(result[0], head.data(), sizeof(int) * cols, TK_MEMCPY_H2D));
    TK_SAFE_CALL(tkMemset(result[1], 0, sizeof(int) * cols));
    TK_SAFE_CALL(tkMemcpy(wall, head.data() + cols, sizeof(int) * (size_t)pyramid_height * cols, TK_MEMCPY_H2D));
    // src = 1, dst = 0 in the reference (src/ori_kernel/path_kernel.cu:139-150): the kernel reads
    // the row that was not copied to and writes over the copied one.  Here the copied row is the
    // source, which is what Rodinia's host loop does on its first step.
    PATHKernelParams = new OriPATHParamsStruct{pyramid_height, wall, result[0], result[1],
                                               cols,           rows, 0,         pyramid_height * PATH_HALO};
    bind();
}

void OriPATHKernel::bind()
{
    OriPATHParamsStruct *q = PATHKernelParams;
    if (q->iteration < 1 || 2 * q->iteration * PATH_HALO >= PATH_BLOCK_SIZE || q->cols < 1)
        logger.ERROR("path: a pyramid of 1 .. 127 rows over at least one column");
    // one block position per PATH_BLOCK_SIZE - 2 * iteration result columns; a wavefront serves it
    // where the reference means a block of PATH_BLOCK_SIZE threads (its launch has grid and block
    // exchanged, src/ori_kernel/path_kernel.cu:136-137)
    launchGridDim = dim3((unsigned)pathBlocks(q->cols, q->iteration), 1, 1);
    launchBlockDim = dim3(TK_WAVE_SIZE, 1, 1);
    kernelParams = {&q->iteration, &q->gpuWall, &q->gpuSrc, &q->gpuResults, &q->cols, &q->rows, &q->startStep, &q->border};
    this->smem = 0;
    auto it = fmap.find("ori_path");
    this->kernelFunc = it == fmap.end() ? nullptr : it->second;
    this->initialized = true;
}

void OriPATHKernel::executeImpl(cudaStream_t stream)
{
    if (!kernelFunc) logger.ERROR("load kernel {ori_path} failed!");
    TK_SAFE_CALL(tkLaunchKernel(this->kernelFunc, launchGridDim.raw(), launchBlockDim.raw(),
                                (void **)this->kernelParams.data(), 0, stream));
}
