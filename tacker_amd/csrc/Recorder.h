// Recorder.h -- per-task table of kernel times (src/Recorder.h of the reference: same
// three calls, same file layout).  One record per task, kernels in the order they ran.
#pragma once
#include <map>
#include <string>
#include <vector>

class Recorder {
public:
    void recordKernel(int taskId, int kernelId, const std::string &kernelName, float executionTime)
    {
        tasks_[taskId].kernels.push_back(KernelTime{kernelId, kernelName, executionTime});
    }
    void recordTask(int taskId, const std::string &taskName) { tasks_[taskId].name = taskName; }
    // Writes the table in the layout of src/Recorder.cc:12-44 (recorder_output.txt):
    //   taskID: <id>, taskName: <name>
    //       kernelID: <id>, kernelName: <name>, execTime: <ms>ms      (one line per kernel)
    //       task running time: <sum>ms
    // and echoes each task header on stdout.  Tasks in ascending id order.
    void text(const std::string &filename = "recorder_output.txt");
    size_t kernelCount(int taskId) { return tasks_[taskId].kernels.size(); }

private:
    struct KernelTime {
        int id;
        std::string name;
        float ms;
    };
    struct TaskTimes {
        std::string name;
        std::vector<KernelTime> kernels;
    };
    std::map<int, TaskTimes> tasks_;
};
