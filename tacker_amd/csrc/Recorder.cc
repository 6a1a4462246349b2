#include "Recorder.h"

#include <fstream>
#include <iostream>

void Recorder::text(const std::string &filename)
{
    std::ofstream file(filename);
    if (!file.is_open()) {
        std::cerr << "cannot open file: " << filename << std::endl;
        return;
    }
    for (auto &task_pair : task_time_map) {
        const int taskId = task_pair.first;
        auto &times = task_pair.second;
        auto &kernelIds = task_kernel_map[taskId];
        auto &taskName = task_name_map[taskId];
        std::cout << "taskID: " << taskId << ", taskName: " << taskName << "\n";
        file << "taskID: " << taskId << ", taskName: " << taskName << "\n";
        float totalTaskTime = 0.0f;
        for (size_t i = 0; i < times.size(); ++i) {
            totalTaskTime += times[i];
            file << "    kernelID: " << kernelIds[i] << ", kernelName: " << task_kernel_name_vec[taskId][i]
                 << ", execTime: " << times[i] << "ms\n";
        }
        file << "    task running time: " << totalTaskTime << "ms\n\n";
    }
}
