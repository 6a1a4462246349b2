// Task.h -- an ordered list of kernels run as one job (src/Task.h of the reference).
#pragma once
#include <string>
#include <vector>

#include "Kernel.h"

enum ExecutionMode { Aker = 0, Tacker };
enum TaskType { LC = 0, BE };

class Task {
public:
    Task(int taskId, std::string taskName);
    explicit Task(int taskId);
    virtual ~Task();
    void addKernel(Kernel *kernel);
    // every kernel in order, each timed with device events; times go to the
    // global Recorder in Aker mode
    void executeTask(ExecutionMode mode, cudaStream_t stream);
    void executeTask(ExecutionMode mode, int idx, cudaStream_t stream);
    // stage the job's input (host -> device copy for a DNN query)
    virtual void initExecution() = 0;
    // the job's launches recorded from `stream` (not the null stream) into one executable graph:
    // every kernel's execute() once, none of them run.  The job must have run before, so that no
    // kernel still has buffers to allocate, and the caller stages the input before each launch of
    // the graph.  The caller destroys the graph (tkGraphExecDestroy).
    tkGraphExec_t captureQuery(cudaStream_t stream);

    int taskId;
    std::string taskName;
    std::vector<Kernel *> kernels;
    TaskType taskType = LC;

    void *Input[3] = {nullptr, nullptr, nullptr};
    void **Result = nullptr;
    void *InputHost[3] = {nullptr, nullptr, nullptr};
    int InputSize[3] = {0, 0, 0};
};
