#include "ModuleCenter.h"

#include <iostream>

#include "Kernel.h"

extern ModuleCenter moduleCenter;

bool Kernel::useModule(const std::string &module, const std::string &function_name)
{
    CUfunction f = moduleCenter.getFunction(module, function_name);
    if (!f) return false;
    function = f;
    moduleName = module;
    launchMode = DRIVER_LAUNCH;
    return true;
}

ModuleCenter::~ModuleCenter()
{
    for (auto &m : modules)
        if (m.second.module) tkModuleUnload(m.second.module);
    modules.clear();
}

bool ModuleCenter::registerModule(const std::string &moduleName, const std::string &codeObjectPath)
{
    if (modules.count(moduleName)) return true;
    ModuleInfo info;
    const int rc = tkModuleLoad(&info.module, codeObjectPath.c_str());
    if (rc != TK_SUCCESS) {
        std::cerr << "Failed to load module from: " << codeObjectPath << " (" << tkGetErrorString(rc)
                  << ")" << std::endl;
        return false;
    }
    modules[moduleName] = info;
    return true;
}

CUfunction ModuleCenter::getFunction(const std::string &moduleName, const std::string &functionName)
{
    auto mit = modules.find(moduleName);
    if (mit == modules.end()) {
        std::cerr << "Module not found: " << moduleName << std::endl;
        return nullptr;
    }
    auto &fns = mit->second.functionMap;
    auto fit = fns.find(functionName);
    if (fit != fns.end()) return fit->second;
    CUfunction f = nullptr;
    if (tkModuleGetFunction(&f, mit->second.module, functionName.c_str()) != TK_SUCCESS) {
        std::cerr << "Function not found in module " << moduleName << ": " << functionName << std::endl;
        return nullptr;
    }
    fns[functionName] = f;
    return f;
}
