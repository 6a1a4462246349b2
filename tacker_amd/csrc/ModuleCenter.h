// ModuleCenter.h -- cache of loaded code objects and their functions.
// Same interface as src/ModuleCenter.h of the reference (registerModule,
// getFunction); modules are gfx950 code objects (.hsaco / .co) loaded through
// tkModuleLoad (hipModuleLoad) instead of cubins through cuModuleLoad.
#pragma once
#include <map>
#include <string>

#include "util.h"

class ModuleCenter {
public:
    ModuleCenter() {}
    ~ModuleCenter();
    // load path under the given name; false (with a message) if it cannot be loaded
    bool registerModule(const std::string &moduleName, const std::string &codeObjectPath);
    // function of a registered module, looked up once and cached; nullptr if absent
    CUfunction getFunction(const std::string &moduleName, const std::string &functionName);

private:
    struct ModuleInfo {
        tkModule_t module = nullptr;
        std::map<std::string, CUfunction> functionMap;
    };
    std::map<std::string, ModuleInfo> modules;
};
