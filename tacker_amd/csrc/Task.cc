#include "Task.h"

#include "Logger.h"
#include "Recorder.h"

extern Logger logger;
extern Recorder recorder;

Task::Task(int taskId, std::string taskName) : taskId(taskId), taskName(std::move(taskName)) {}
Task::Task(int taskId) : taskId(taskId) {}

Task::~Task()
{
    logger.DEBUG("task name: " + taskName + ", id: " + std::to_string(taskId) + " is destroyed!");
}

void Task::addKernel(Kernel *kernel) { kernels.emplace_back(kernel); }

namespace {
struct EventPair {
    tkEvent_t start = nullptr, stop = nullptr;
    EventPair()
    {
        TK_SAFE_CALL(tkEventCreate(&start));
        TK_SAFE_CALL(tkEventCreate(&stop));
    }
    ~EventPair()
    {
        tkEventDestroy(start);
        tkEventDestroy(stop);
    }
    float time(Kernel *kernel, cudaStream_t stream)
    {
        float ms = 0.0f;
        TK_SAFE_CALL(tkEventRecord(start, stream));
        kernel->execute(stream);
        TK_SAFE_CALL(tkEventRecord(stop, stream));
        TK_SAFE_CALL(tkEventSynchronize(stop));
        TK_SAFE_CALL(tkEventElapsedTime(&ms, start, stop));
        return ms;
    }
};
}  // namespace

void Task::executeTask(ExecutionMode mode, cudaStream_t stream)
{
    EventPair ev;
    for (auto &kernel : kernels) {
        logger.DEBUG("kernel name: " + kernel->kernelName + ", id: " + std::to_string(kernel->Id) + " is executing ...");
        const float kernel_time = ev.time(kernel, stream);
        if (mode == ExecutionMode::Aker) recorder.recordKernel(taskId, kernel->Id, kernel->kernelName, kernel_time);
    }
    if (mode == ExecutionMode::Aker) recorder.recordTask(taskId, taskName);
}

tkGraphExec_t Task::captureQuery(cudaStream_t stream)
{
    tkGraphExec_t graph = nullptr;
    TK_SAFE_CALL(tkStreamBeginCapture(stream));
    try {
        for (auto &kernel : kernels) kernel->execute(stream);
    } catch (...) {   // a stream left recording would fail every later call on it
        tkStreamEndCapture(stream, &graph);
        if (graph) tkGraphExecDestroy(graph);
        throw;
    }
    TK_SAFE_CALL(tkStreamEndCapture(stream, &graph));
    return graph;
}

void Task::executeTask(ExecutionMode mode, int idx, cudaStream_t stream)
{
    EventPair ev;
    Kernel *kernel = this->kernels.at(idx);
    const float kernel_time = ev.time(kernel, stream);
    if (mode == ExecutionMode::Aker) recorder.recordKernel(taskId, kernel->Id, kernel->kernelName, kernel_time);
}
