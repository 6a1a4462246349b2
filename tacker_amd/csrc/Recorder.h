// Recorder.h -- per-task kernel-time table (src/Recorder.h of the reference).
#pragma once
#include <string>
#include <unordered_map>
#include <vector>

class Recorder {
public:
    void recordKernel(int taskId, int kernelId, const std::string &kernelName, float executionTime)
    {
        task_time_map[taskId].push_back(executionTime);
        task_kernel_map[taskId].push_back(kernelId);
        task_kernel_name_vec[taskId].push_back(kernelName);
    }
    void recordTask(int taskId, const std::string &taskName) { task_name_map[taskId] = taskName; }
    // writes recorder_output.txt in the layout of src/Recorder.cc:12-44
    void text(const std::string &filename = "recorder_output.txt");
    size_t kernelCount(int taskId) { return task_time_map[taskId].size(); }

private:
    std::unordered_map<int, std::vector<float>> task_time_map;
    std::unordered_map<int, std::vector<int>> task_kernel_map;
    std::unordered_map<int, std::vector<std::string>> task_kernel_name_vec;
    std::unordered_map<int, std::string> task_name_map;
};
