// aker -- the command line of the reference (src/main.cu:227-300):
//   aker -s <aker|tacker> -m <model> [-d <device>] [-c <kinfo.json>]
// loads the kernel-info table, brings the device up, prints build and device facts, builds
// the latency-critical task, warms it up (5 queries), names the two best-effort kernels of
// kinfo's "throughput_test" entry ("[Result] cd1: .., cd2: .., dnn: .."), and runs
// TaskManager::executeAllTasks in Aker and then in Tacker mode, whose "[PRE]", "[Ori]",
// "[Mix]" and "[Result]" lines are what the reference's scripts scrape.  At exit the
// recorder's table goes to recorder_output.txt (my_exit, src/main.cu:203-206); one recorded
// pass of the task fills it (the reference's live main records nothing, so its file is empty).
// -c is an addition: without it the table built into the library is used instead of
// <ROOT>/config/kinfo-<model>.json.
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <iostream>
#include <string>

#include "Creator.h"
#include "Logger.h"
#include "Recorder.h"
#include "Task.h"
#include "TaskManager.h"
#include "dnn/vgg16.h"
#include "json.h"

extern Logger logger;
extern Recorder recorder;
int tacker_runtime_init(int device, const char *kinfo_json_path);

#define AKER_VERSION_MAJOR 1
#define AKER_VERSION_MINOR 0
#define AKER_VERSION_PATCH 0

namespace {

void usage(const char *program)
{
    std::cout << "SYNOPSIS\n        " << program
              << " -s <system_name> -m <model_name> [-d <device_no>] [-c <kinfo.json>]\n\n"
              << "OPTIONS\n"
              << "        -s, --system <system_name>   system name, aker/tacker\n"
              << "        -m, --model <model_name>     model name\n"
              << "        -d, --device <device_no>     device number\n"
              << "        -c, --config <kinfo.json>    kernel-info table (default: the built-in one)\n";
}

void compileInfo()
{
    std::cout << "Acker Version: " << AKER_VERSION_MAJOR << "." << AKER_VERSION_MINOR << "." << AKER_VERSION_PATCH
              << std::endl;
    std::cout << "Compile Timestamp: " << __DATE__ << " " << __TIME__ << std::endl;
}

// the device facts the reference prints (src/main.cu:185-201), for this device layer
void printDeviceProp()
{
    int cus = 0;
    char name[256] = "";
    tkGetCuCount(&cus);
    tkGetDeviceName(name, sizeof(name));
    std::cout << "device\t\t\t" << name << std::endl;
    std::cout << "SM num\t\t\t" << cus << std::endl;
    std::cout << "max threads per blk\t" << 1024 << std::endl;
    std::cout << "warp size\t\t" << 64 << std::endl;
    std::cout << "shared memory\t\t" << 160 * 1024 << std::endl;
}

void my_exit()
{
    recorder.text();
    logger.INFO("System exit");
}

}  // namespace

int main(int argc, char *argv[])
{
    std::string system_name, model_name, config_path;
    int device_no = 0;
    bool ok = true;
    for (int i = 1; i < argc && ok; ++i) {
        const std::string a = argv[i];
        const bool has_value = i + 1 < argc;
        if ((a == "-s" || a == "--system") && has_value) system_name = argv[++i];
        else if ((a == "-m" || a == "--model") && has_value) model_name = argv[++i];
        else if ((a == "-d" || a == "--device") && has_value) device_no = std::atoi(argv[++i]);
        else if ((a == "-c" || a == "--config") && has_value) config_path = argv[++i];
        else ok = false;
    }
    if (!ok || system_name.empty() || model_name.empty()) {
        usage(argv[0]);
        return 0;
    }
    std::cout << "system: " << system_name << ", model: " << model_name << std::endl;

    std::atexit(my_exit);

    const int rc = tacker_runtime_init(device_no, config_path.empty() ? nullptr : config_path.c_str());
    if (rc) logger.ERROR(std::string("device init failed: ") + tkGetErrorString(rc));
    logger.INFO("device init complete!");
    compileInfo();
    printDeviceProp();

    tkStream_t streams[2];
    TK_SAFE_CALL(tkStreamCreate(&streams[0]));
    TK_SAFE_CALL(tkStreamCreate(&streams[1]));

    Task *lc_task = createTask(model_name);
    for (int i = 0; i < 5; ++i) {
        lc_task->initExecution();
        for (auto &kernel : lc_task->kernels) kernel->execute(nullptr);
        TK_SAFE_CALL(tkDeviceSynchronize());
    }
    lc_task->initExecution();
    lc_task->executeTask(ExecutionMode::Aker, streams[0]);   // the recorder's table

    const std::string a = sget_kernel_info("throughput_test", "a");
    const std::string b = sget_kernel_info("throughput_test", "b");
    std::printf("[Result] cd1: %s, cd2: %s, dnn: %s\n", a.c_str(), b.c_str(), model_name.c_str());
    TaskManager taskManager(lc_task, a, b);
    taskManager.executeAllTasks(ExecutionMode::Aker, streams[0]);
    taskManager.executeAllTasks(ExecutionMode::Tacker, streams[1]);

    TK_SAFE_CALL(tkDeviceSynchronize());
    TK_SAFE_CALL(tkStreamDestroy(streams[0]));
    TK_SAFE_CALL(tkStreamDestroy(streams[1]));
    std::fflush(stdout);
    return 0;
}
