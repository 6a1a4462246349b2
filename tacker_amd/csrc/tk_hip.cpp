// tk_hip.cpp -- the HIP implementation of the thin device layer (tk*).
// One function per CUDA runtime / driver call the reference's host code makes;
// HIP error codes are folded into TK_ERROR_DEVICE with the HIP text kept for
// tkGetErrorString.
#include <hip/hip_runtime.h>

#include <atomic>

#include <cstring>
#include <mutex>
#include <string>
#include <vector>

#include "../../include/tacker_amd.h"

extern "C" int tk_device_symbol(const char *name, const void **symbol, size_t *bytes);
extern "C" int tk_scratch_setup(int device);

namespace {
thread_local std::string g_last_hip_error;
std::mutex g_modules_mutex;
std::vector<hipModule_t> g_modules;   // code objects loaded through tkModuleLoad
const char *const kMirroredSymbols[] = {"ck", "c_mrif", "atominfo", "NbrListLen", "NbrList", "tz_ws_table", "tk_spin_fail"};

int fold(hipError_t e, const char *what)
{
    if (e == hipSuccess) return TK_SUCCESS;
    g_last_hip_error = std::string(what) + ": " + hipGetErrorString(e);
    (void)hipGetLastError();   // clear the sticky error
    return TK_ERROR_DEVICE;
}
hipMemcpyKind kind_of(int kind)
{
    switch (kind) {
        case TK_MEMCPY_H2D: return hipMemcpyHostToDevice;
        case TK_MEMCPY_D2H: return hipMemcpyDeviceToHost;
        case TK_MEMCPY_D2D: return hipMemcpyDeviceToDevice;
        default: return hipMemcpyDefault;
    }
}
}  // namespace

#define FOLD(call) fold((call), #call)

extern "C" {

int tkInit(int device)
{
    int count = 0;
    int rc = FOLD(hipGetDeviceCount(&count));
    if (rc) return rc;
    if (device < 0 || device >= count) {
        g_last_hip_error = "tkInit: no such device";
        return TK_ERROR_INVALID_VALUE;
    }
    rc = FOLD(hipSetDevice(device));
    if (rc) return rc;
    rc = FOLD(hipFree(0));   // force context creation, as initCUDA does
    if (rc) return rc;
    rc = tk_scratch_setup(device);   // device address of the library's static scratch array
    if (rc) g_last_hip_error = "tkInit: hipGetSymbolAddress of the static scratch array failed";
    return rc;
}

const char *tkGetErrorString(int code)
{
    switch (code) {
        case TK_SUCCESS: return "success";
        case TK_ERROR_INVALID_VALUE: return g_last_hip_error.empty() ? "invalid value" : g_last_hip_error.c_str();
        case TK_ERROR_NOT_FOUND: return "not found";
        case TK_ERROR_UNSUPPORTED: return "unsupported shape";
        case TK_ERROR_DEVICE: return g_last_hip_error.c_str();
        default: return "unknown error";
    }
}

int tkGetCuCount(int *cu_count)
{
    int dev = 0;
    int rc = FOLD(hipGetDevice(&dev));
    if (rc) return rc;
    return FOLD(hipDeviceGetAttribute(cu_count, hipDeviceAttributeMultiprocessorCount, dev));
}

int tkGetDeviceName(char *buf, size_t len)
{
    int dev = 0;
    int rc = FOLD(hipGetDevice(&dev));
    if (rc) return rc;
    hipDeviceProp_t prop;
    rc = FOLD(hipGetDeviceProperties(&prop, dev));
    if (rc) return rc;
    snprintf(buf, len, "%s (%s)", prop.name, prop.gcnArchName);
    return TK_SUCCESS;
}

// calls of tkMalloc / tkFree since the library was loaded: what a caller that must not allocate
// (a captured graph, a serving loop) checks around a call
static std::atomic<long long> g_malloc_calls{0}, g_free_calls{0};
int tkMalloc(void **ptr, size_t bytes)
{
    ++g_malloc_calls;
    return FOLD(hipMalloc(ptr, bytes));
}
int tkFree(void *ptr)
{
    ++g_free_calls;
    return FOLD(hipFree(ptr));
}
int tkAllocationCalls(long long *mallocs, long long *frees)
{
    if (mallocs) *mallocs = g_malloc_calls.load();
    if (frees) *frees = g_free_calls.load();
    return TK_SUCCESS;
}
int tkMemcpy(void *dst, const void *src, size_t bytes, int kind)
{
    return FOLD(hipMemcpy(dst, src, bytes, kind_of(kind)));
}
int tkMemcpyAsync(void *dst, const void *src, size_t bytes, int kind, tkStream_t s)
{
    return FOLD(hipMemcpyAsync(dst, src, bytes, kind_of(kind), (hipStream_t)s));
}
int tkMemset(void *ptr, int value, size_t bytes) { return FOLD(hipMemset(ptr, value, bytes)); }

int tkMemcpyToSymbol(const char *symbol, const void *src, size_t bytes, size_t offset)
{
    const void *sym = nullptr;
    size_t cap = 0;
    const int rc = tk_device_symbol(symbol, &sym, &cap);
    if (rc) return rc;
    if (offset + bytes > cap) {
        g_last_hip_error = "tkMemcpyToSymbol: range exceeds the symbol";
        return TK_ERROR_INVALID_VALUE;
    }
    const int wrote = FOLD(hipMemcpyToSymbol(sym, src, bytes, offset, hipMemcpyHostToDevice));
    if (wrote) return wrote;
    std::lock_guard<std::mutex> lock(g_modules_mutex);
    for (hipModule_t mod : g_modules) {   // the loaded code objects' copies follow
        hipDeviceptr_t dst = nullptr;
        size_t have = 0;
        if (hipModuleGetGlobal(&dst, &have, mod, symbol) != hipSuccess) {
            (void)hipGetLastError();
            continue;
        }
        if (offset + bytes > have) continue;
        const int e = FOLD(hipMemcpy((char *)dst + offset, src, bytes, hipMemcpyHostToDevice));
        if (e) return e;
    }
    return TK_SUCCESS;
}

int tkMemcpyFromSymbol(void *dst, const char *symbol, size_t bytes, size_t offset)
{
    const void *sym = nullptr;
    size_t cap = 0;
    const int rc = tk_device_symbol(symbol, &sym, &cap);
    if (rc) return rc;
    if (offset + bytes > cap) {
        g_last_hip_error = "tkMemcpyFromSymbol: range exceeds the symbol";
        return TK_ERROR_INVALID_VALUE;
    }
    const int got = FOLD(hipMemcpyFromSymbol(dst, sym, bytes, offset, hipMemcpyDeviceToHost));
    if (got || strcmp(symbol, "tk_spin_fail") != 0 || bytes != sizeof(unsigned) || offset != 0) return got;
    // the failure word is a set of bits any kernel may raise: those of loaded code objects count too
    std::lock_guard<std::mutex> lock(g_modules_mutex);
    for (hipModule_t mod : g_modules) {
        hipDeviceptr_t src = nullptr;
        size_t have = 0;
        unsigned bits = 0;
        if (hipModuleGetGlobal(&src, &have, mod, symbol) != hipSuccess) {
            (void)hipGetLastError();
            continue;
        }
        const int e = FOLD(hipMemcpy(&bits, src, sizeof(bits), hipMemcpyDeviceToHost));
        if (e) return e;
        *(unsigned *)dst |= bits;
    }
    return TK_SUCCESS;
}

int tkStreamCreate(tkStream_t *s) { return FOLD(hipStreamCreate((hipStream_t *)s)); }
int tkStreamDestroy(tkStream_t s) { return FOLD(hipStreamDestroy((hipStream_t)s)); }
int tkStreamSynchronize(tkStream_t s) { return FOLD(hipStreamSynchronize((hipStream_t)s)); }
int tkDeviceSynchronize(void) { return FOLD(hipDeviceSynchronize()); }
int tkEventCreate(tkEvent_t *e) { return FOLD(hipEventCreate((hipEvent_t *)e)); }
int tkEventDestroy(tkEvent_t e) { return FOLD(hipEventDestroy((hipEvent_t)e)); }
int tkStreamBeginCapture(tkStream_t s)
{
    if (!s) return TK_ERROR_INVALID_VALUE;   // the null stream cannot be captured
    return FOLD(hipStreamBeginCapture((hipStream_t)s, hipStreamCaptureModeThreadLocal));
}
int tkStreamEndCapture(tkStream_t s, tkGraphExec_t *exec)
{
    if (!s || !exec) return TK_ERROR_INVALID_VALUE;
    hipGraph_t graph = nullptr;
    int rc = FOLD(hipStreamEndCapture((hipStream_t)s, &graph));
    if (rc) return rc;
    hipGraphExec_t made = nullptr;
    rc = FOLD(hipGraphInstantiate(&made, graph, nullptr, nullptr, 0));
    (void)hipGraphDestroy(graph);
    if (rc) return rc;
    *exec = made;
    return TK_SUCCESS;
}
int tkGraphLaunch(tkGraphExec_t exec, tkStream_t s)
{
    if (!exec) return TK_ERROR_INVALID_VALUE;
    return FOLD(hipGraphLaunch((hipGraphExec_t)exec, (hipStream_t)s));
}
int tkGraphExecDestroy(tkGraphExec_t exec) { return exec ? FOLD(hipGraphExecDestroy((hipGraphExec_t)exec)) : TK_SUCCESS; }
int tkEventRecord(tkEvent_t e, tkStream_t s) { return FOLD(hipEventRecord((hipEvent_t)e, (hipStream_t)s)); }
int tkEventSynchronize(tkEvent_t e) { return FOLD(hipEventSynchronize((hipEvent_t)e)); }
int tkEventElapsedTime(float *ms, tkEvent_t start, tkEvent_t stop)
{
    return FOLD(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
}

int tkLaunchKernel(const void *func, tkDim3 grid, tkDim3 block, void **args, size_t shmem,
                   tkStream_t stream)
{
    if (!func) {
        g_last_hip_error = "tkLaunchKernel: null function";
        return TK_ERROR_INVALID_VALUE;
    }
    return FOLD(hipLaunchKernel(func, dim3(grid.x, grid.y, grid.z), dim3(block.x, block.y, block.z),
                                args, shmem, (hipStream_t)stream));
}

// A code object carries copies of its own of the device symbols the host fills by name (constant
// tables, the workspace table, the failure word).  They follow the library's: filled from the
// library's copies when the object is loaded, and written along with them from then on.
int tkModuleLoad(tkModule_t *m, const char *path)
{
    hipModule_t mod = nullptr;
    const int rc = FOLD(hipModuleLoad(&mod, path));
    if (rc) return rc;
    for (const char *name : kMirroredSymbols) {
        hipDeviceptr_t dst = nullptr;
        size_t bytes = 0;
        if (hipModuleGetGlobal(&dst, &bytes, mod, name) != hipSuccess) {
            (void)hipGetLastError();   // this object does not use the symbol
            continue;
        }
        const void *sym = nullptr;
        void *src = nullptr;
        size_t cap = 0;
        int e = tk_device_symbol(name, &sym, &cap);
        if (!e) e = FOLD(hipGetSymbolAddress(&src, sym));
        if (!e) e = FOLD(hipMemcpy(dst, src, bytes < cap ? bytes : cap, hipMemcpyDeviceToDevice));
        if (e) {
            (void)hipModuleUnload(mod);
            return e;
        }
    }
    std::lock_guard<std::mutex> lock(g_modules_mutex);
    g_modules.push_back(mod);
    *m = mod;
    return TK_SUCCESS;
}
int tkModuleUnload(tkModule_t m)
{
    {
        std::lock_guard<std::mutex> lock(g_modules_mutex);
        for (size_t i = 0; i < g_modules.size(); ++i)
            if (g_modules[i] == (hipModule_t)m) {
                g_modules.erase(g_modules.begin() + (long)i);
                break;
            }
    }
    return FOLD(hipModuleUnload((hipModule_t)m));
}
int tkModuleGetFunction(tkFunction_t *f, tkModule_t m, const char *name)
{
    return FOLD(hipModuleGetFunction((hipFunction_t *)f, (hipModule_t)m, name));
}
int tkModuleLaunchKernel(tkFunction_t f, tkDim3 grid, tkDim3 block, void **args, size_t shmem,
                         tkStream_t stream)
{
    return FOLD(hipModuleLaunchKernel((hipFunction_t)f, grid.x, grid.y, grid.z, block.x, block.y,
                                      block.z, (unsigned)shmem, (hipStream_t)stream, args, nullptr));
}

}  // extern "C"
