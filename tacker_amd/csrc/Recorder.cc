#include "Recorder.h"

#include <cstdio>
#include <sstream>

void Recorder::text(const std::string &filename)
{
    // numbers print the way the reference's stream insertion prints a float (%g, 6 digits)
    std::ostringstream table;
    for (const auto &entry : tasks_) {
        const TaskTimes &task = entry.second;
        std::ostringstream header;
        header << "taskID: " << entry.first << ", taskName: " << task.name << "\n";
        std::fputs(header.str().c_str(), stdout);
        table << header.str();
        float total = 0.0f;
        for (const KernelTime &k : task.kernels) {
            table << "    kernelID: " << k.id << ", kernelName: " << k.name << ", execTime: " << k.ms << "ms\n";
            total += k.ms;
        }
        table << "    task running time: " << total << "ms\n\n";
    }
    FILE *file = std::fopen(filename.c_str(), "w");
    if (!file) {
        std::fprintf(stderr, "cannot open file: %s\n", filename.c_str());
        return;
    }
    std::fputs(table.str().c_str(), file);
    std::fclose(file);
}
