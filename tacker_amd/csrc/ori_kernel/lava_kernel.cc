#include "lava_kernel.h"

#include <unordered_map>

#include "../Logger.h"
#include "fill.h"

extern Logger logger;
extern std::unordered_map<std::string, void *> fmap;

std::vector<box_str> lavaBoxes(int boxes1d)
{
    std::vector<box_str> boxes((size_t)boxes1d * boxes1d * boxes1d, box_str{});
    int nh = 0;
    for (int z = 0; z < boxes1d; ++z)
        for (int y = 0; y < boxes1d; ++y)
            for (int x = 0; x < boxes1d; ++x, ++nh) {
                box_str &b = boxes[nh];
                b.x = x, b.y = y, b.z = z;
                b.number = nh;
                b.offset = (long)nh * NUMBER_PAR_PER_BOX;
                b.nn = 0;
                for (int dz = -1; dz <= 1; ++dz)
                    for (int dy = -1; dy <= 1; ++dy)
                        for (int dx = -1; dx <= 1; ++dx) {
                            const int nx = x + dx, ny = y + dy, nz = z + dz;
                            const bool inside = nx >= 0 && ny >= 0 && nz >= 0 && nx < boxes1d && ny < boxes1d && nz < boxes1d;
                            if (!inside || (dx == 0 && dy == 0 && dz == 0)) continue;
                            nei_str &n = b.nei[b.nn++];
                            n.x = nx, n.y = ny, n.z = nz;
                            n.number = nz * boxes1d * boxes1d + ny * boxes1d + nx;
                            n.offset = (long)n.number * NUMBER_PAR_PER_BOX;
                        }
            }
    return boxes;
}

OriLAVAKernel::OriLAVAKernel(int id)
{
    Id = id;
    this->kernelName = "lava";
    initParams();
}

OriLAVAKernel::OriLAVAKernel(int id, float alpha, int boxes1d, FOUR_VECTOR *rv, float *qv, FOUR_VECTOR *fv)
{
    Id = id;
    this->kernelName = "lava";
    bind(alpha, boxes1d, rv, qv, fv);
}

OriLAVAKernel::~OriLAVAKernel()
{
    for (auto &ptr : cudaFreeList) tkErrCheck(tkFree(ptr));
    delete LAVAKernelParams;
}

void OriLAVAKernel::initParams()
{
    const int boxes1d = 60;
    const size_t particles = (size_t)boxes1d * boxes1d * boxes1d * NUMBER_PAR_PER_BOX;
    FOUR_VECTOR *rv = nullptr, *fv = nullptr;
    float *qv = nullptr;
    TK_SAFE_CALL(tkMalloc((void **)&rv, particles * sizeof(FOUR_VECTOR)));
    cudaFreeList.push_back(rv);
    TK_SAFE_CALL(tkMalloc((void **)&qv, particles * sizeof(float)));
    cudaFreeList.push_back(qv);
    TK_SAFE_CALL(tkMalloc((void **)&fv, particles * sizeof(FOUR_VECTOR)));
    cudaFreeList.push_back(fv);
    tkFillUniform(reinterpret_cast<float *>(rv), 4 * particles, 4301u, 0.1f, 1.0f);
    tkFillUniform(qv, particles, 4302u, 0.1f, 1.0f);
    TK_SAFE_CALL(tkMemset(fv, 0, particles * sizeof(FOUR_VECTOR)));
    bind(0.5f, boxes1d, rv, qv, fv);
}

void OriLAVAKernel::bind(float alpha, int boxes1d, FOUR_VECTOR *rv, float *qv, FOUR_VECTOR *fv)
{
    if (boxes1d < 1 || boxes1d > 128) logger.ERROR("lava: 1 .. 128 boxes along an edge");
    const std::vector<box_str> boxes = lavaBoxes(boxes1d);
    box_str *d_box = nullptr;
    TK_SAFE_CALL(tkMalloc((void **)&d_box, boxes.size() * sizeof(box_str)));
    cudaFreeList.push_back(d_box);
    TK_SAFE_CALL(tkMemcpy(d_box, boxes.data(), boxes.size() * sizeof(box_str), TK_MEMCPY_H2D));
    LAVAKernelParams = new OriLAVAParamsStruct{};
    OriLAVAParamsStruct *q = LAVAKernelParams;
    q->d_par_gpu.alpha = alpha;
    q->d_dim_gpu.boxes1d_arg = boxes1d;
    q->d_dim_gpu.number_boxes = (long)boxes.size();
    q->d_dim_gpu.space_elem = q->d_dim_gpu.number_boxes * NUMBER_PAR_PER_BOX;
    q->d_dim_gpu.space_mem = q->d_dim_gpu.space_elem * (long)sizeof(FOUR_VECTOR);
    q->d_dim_gpu.space_mem2 = q->d_dim_gpu.space_elem * (long)sizeof(float);
    q->d_dim_gpu.box_mem = q->d_dim_gpu.number_boxes * (long)sizeof(box_str);
    q->d_box_gpu = d_box;
    q->d_rv_gpu = rv;
    q->d_qv_gpu = qv;
    q->d_fv_gpu = fv;
    // the reference's grid is one block per box (src/ori_kernel/lava_kernel.cu:275-278); the position
    // grid has the 27 parts of a box's work as a second dimension, and a wavefront serves a box where
    // the reference launches 128 threads
    launchGridDim = dim3((unsigned)boxes.size(), 1, LAVA_PARTS);
    launchBlockDim = dim3(TK_WAVE_SIZE, 1, 1);
    kernelParams = {&q->d_par_gpu, &q->d_dim_gpu, &q->d_box_gpu, &q->d_rv_gpu, &q->d_qv_gpu, &q->d_fv_gpu};
    this->smem = 0;
    auto it = fmap.find("ori_lava");
    this->kernelFunc = it == fmap.end() ? nullptr : it->second;
    this->initialized = true;
}

void OriLAVAKernel::executeImpl(cudaStream_t stream)
{
    if (!kernelFunc) logger.ERROR("load kernel {ori_lava} failed!");
    // every box through all its parts: one wavefront per box
    TK_SAFE_CALL(tkLaunchKernel(this->kernelFunc, dim3(launchGridDim.x, 1, 1).raw(), launchBlockDim.raw(),
                                (void **)this->kernelParams.data(), 0, stream));
}
