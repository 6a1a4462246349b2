#include "fill.h"

#include <string>
#include <unordered_map>

#include "../Logger.h"
#include "../util.h"

extern Logger logger;
extern std::unordered_map<std::string, void *> fmap;

static void launchFill(const char *key, void **args, size_t n)
{
    auto it = fmap.find(key);
    if (it == fmap.end()) logger.ERROR(std::string("load kernel {") + key + "} failed!");
    if (n == 0) return;
    const size_t blocks = (n + 255) / 256;
    const unsigned grid = (unsigned)(blocks < 65536 ? blocks : 65536);   // the kernels stride over the rest
    TK_SAFE_CALL(tkLaunchKernel(it->second, dim3(grid, 1, 1).raw(), dim3(256, 1, 1).raw(), args, 0, nullptr));
    TK_SAFE_CALL(tkDeviceSynchronize());
}

void tkFillUniform(float *dst, size_t n, unsigned seed, float lo, float hi)
{
    unsigned long long count = n;
    void *args[] = {&dst, &count, &seed, &lo, &hi};
    launchFill("fill_uniform", args, n);
}

void tkFillIntMod(int *dst, size_t n, unsigned seed, int mod)
{
    unsigned long long count = n;
    void *args[] = {&dst, &count, &seed, &mod};
    launchFill("fill_int_mod", args, n);
}
