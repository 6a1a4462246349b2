// OriNNKernel -- host object of Rodinia's nearest-neighbour distance kernel
// (src/ori_kernel/nn_kernel.{h,cu} of the reference).
#pragma once
#include "../Kernel.h"
#include "../header/nn_header.h"

struct OriNNParamsStruct {
    LatLong *d_locations;
    float *d_distances;
    int numRecords;
    float lat;
    float lng;
};

class OriNNKernel : public Kernel {
public:
    // 256 * 2560000 records (src/ori_kernel/nn_kernel.cu:46).  The reference copies its records
    // from an empty vector and never sets the query point; here the records are filled on the
    // device, latitude and longitude uniform in [0, 90) (tkFillUniform with seed 4001 over the
    // interleaved array), and the query is Rodinia's example (30, 90).
    explicit OriNNKernel(int id);
    // caller-owned records and distances
    OriNNKernel(int id, LatLong *d_locations, float *d_distances, int numRecords, float lat, float lng);
    ~OriNNKernel() override;

    void initParams() override;
    std::vector<int> getArgs() override { return std::vector<int>(); }
    OriNNParamsStruct *params() { return NNKernelParams; }

protected:
    void executeImpl(cudaStream_t stream) override;

private:
    void loadKernel() override {}
    void bind();
    OriNNParamsStruct *NNKernelParams = nullptr;
};

// blocks of NN_THREADS_PER_BLOCK records (the reference's ceilDiv, src/ori_kernel/nn_kernel.cu:74)
int nnBlocks(int numRecords);
