// runtime.cc -- process-wide state of the host runtime: the objects the
// reference defines in src/main.cu (logger, recorder, moduleCenter, fmap) and in
// src/TaskManager.cu:19-46 (global GEMM buffers), and the one-time set-up.
#include <mutex>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

#include "Logger.h"
#include "ModuleCenter.h"
#include "Recorder.h"
#include "json.h"
#include "rng.h"
#include "tzgemm_kernel.h"
#include "ori_kernel/sgemm_kernel.h"
#include "mix_kernel/kinfo_builtin.inc"

Logger logger("", getenv("TACKER_QUIET") == nullptr, false);
Recorder recorder;
ModuleCenter moduleCenter;
std::unordered_map<std::string, void *> fmap;

long long MAX_ORI_WMMA_A = 0;
long long MAX_ORI_WMMA_B = 0;
long long MAX_ORI_WMMA_C = 0;
bool gemm_malloced = false;
void *ori_wmma_A = nullptr;
void *ori_wmma_B = nullptr;
float *ori_wmma_C = nullptr;

static void grow(void **ptr, long long *have, long long need, bool seed_halves)
{
    if (need <= *have) return;
    TK_SAFE_CALL(tkDeviceSynchronize());   // nothing may still be using the old buffer
    if (*ptr) TK_SAFE_CALL(tkFree(*ptr));
    TK_SAFE_CALL(tkMalloc(ptr, (size_t)need));
    *have = need;
    if (seed_halves) {
        std::vector<uint16_t> host((size_t)need / 2);
        tk::Rng rng(1337ULL + (uint64_t)need);
        for (auto &h : host) h = tk::float_to_half_bits(rng.uniform(-1.0f, 1.0f));
        TK_SAFE_CALL(tkMemcpy(*ptr, host.data(), (size_t)need, TK_MEMCPY_H2D));
    } else {
        TK_SAFE_CALL(tkMemset(*ptr, 0, (size_t)need));
        TK_SAFE_CALL(tkDeviceSynchronize());   // zero before a kernel on any stream touches it
    }
}

void ensureGlobalGemmBuffers(int M_GLOBAL, int N_GLOBAL, int K_GLOBAL)
{
    const long long a = 2LL * M_GLOBAL * K_GLOBAL;
    const long long b = 2LL * N_GLOBAL * K_GLOBAL;
    const long long c = 4LL * M_GLOBAL * N_GLOBAL;
    if (!gemm_malloced)
        logger.INFO("[ori_tzgemm][initParams] allocating global GEMM buffers A " + std::to_string(a >> 20) +
                    " MB, B " + std::to_string(b >> 20) + " MB, C " + std::to_string(c >> 20) + " MB");
    grow(&ori_wmma_A, &MAX_ORI_WMMA_A, a, true);
    grow(&ori_wmma_B, &MAX_ORI_WMMA_B, b, true);
    grow((void **)&ori_wmma_C, &MAX_ORI_WMMA_C, c, false);
    gemm_malloced = true;
}

namespace {
struct BoundWorkspace {
    void *ptr;
    long long bytes;
    bool zero_at_rest;   // only kernels that hand it back all zero (tzgemm's counters) have used it
};
std::mutex g_workspace_mutex;
std::unordered_map<const void *, BoundWorkspace> g_workspaces;   // by output buffer
std::vector<void *> g_outgrown_workspaces;   // replaced by a larger one; launches in flight may still use them
constexpr size_t kMaxBoundWorkspaces = TZ_WS_TABLE_SLOTS / 2;   // load factor of the device table
std::vector<tz_ws_entry> g_table_mirror(TZ_WS_TABLE_SLOTS, tz_ws_entry{0, 0});   // host copy of tz_ws_table

// Enters (C, workspace) into the device table, or updates C's entry.  A slot is written with one
// 16-byte copy and never moves, so a kernel that runs meanwhile and probes past it for another key
// sees it either empty or whole.
void publish_workspace(const void *C, void *workspace)
{
    const unsigned long long key = (unsigned long long)(size_t)C;
    unsigned slot = tz_ws_hash(key);
    for (int probe = 0; probe < TZ_WS_TABLE_MAX_PROBES; ++probe, slot = (slot + 1) & (TZ_WS_TABLE_SLOTS - 1)) {
        if (g_table_mirror[slot].c != key && g_table_mirror[slot].c != 0) continue;
        g_table_mirror[slot] = tz_ws_entry{key, (unsigned long long)(size_t)workspace};
        TK_SAFE_CALL(tkMemcpyToSymbol("tz_ws_table", &g_table_mirror[slot], sizeof(tz_ws_entry),
                                      slot * sizeof(tz_ws_entry)));
        return;
    }
    throw std::runtime_error("tzgemm: the device table of workspaces has no free slot near this output "
                             "buffer's hash; call tzgemmReleaseWorkspaces() once the kernels that use them are gone");
}
}  // namespace

// A device buffer of at least `need` bytes bound to the output buffer C.  keeps_zero: the asking
// kernel needs it zero and leaves it zero (tzgemm's arrival counters); sgemm writes its partial sums
// before it reads them and leaves them there, so a buffer it has used is cleared again before a
// kernel of the first kind gets it (an output address the caller's allocator handed out twice).
static void *workspaceFor(const void *C, long long need, bool keeps_zero)
{
    if (need == 0 || C == nullptr) return nullptr;
    std::lock_guard<std::mutex> lock(g_workspace_mutex);
    auto it = g_workspaces.find(C);
    if (it != g_workspaces.end() && it->second.bytes >= need) {
        if (keeps_zero && !it->second.zero_at_rest) {
            TK_SAFE_CALL(tkDeviceSynchronize());   // the kernels that wrote it are done
            TK_SAFE_CALL(tkMemset(it->second.ptr, 0, (size_t)it->second.bytes));
            TK_SAFE_CALL(tkDeviceSynchronize());
            it->second.zero_at_rest = true;
        }
        if (!keeps_zero) it->second.zero_at_rest = false;
        return it->second.ptr;
    }
    if (it == g_workspaces.end() && g_workspaces.size() >= kMaxBoundWorkspaces)
        throw std::runtime_error("tzgemm: " + std::to_string(kMaxBoundWorkspaces) +
                                 " output buffers hold a workspace; call tzgemmReleaseWorkspaces() once the "
                                 "kernels that use them are gone");
    // a new binding is rare (first kernel object on this C, or a larger shape), so it may wait for the device
    void *ptr = nullptr;
    TK_SAFE_CALL(tkMalloc(&ptr, (size_t)need));
    TK_SAFE_CALL(tkMemset(ptr, 0, (size_t)need));
    TK_SAFE_CALL(tkDeviceSynchronize());   // zero before any stream's kernel reads the counters
    try {
        publish_workspace(C, ptr);
    } catch (...) {
        tkErrCheck(tkFree(ptr));
        throw;
    }
    if (it != g_workspaces.end()) g_outgrown_workspaces.push_back(it->second.ptr);
    g_workspaces[C] = BoundWorkspace{ptr, need, keeps_zero};
    return ptr;
}

void *tzgemmWorkspaceFor(const float *C, int M_GLOBAL, int N_GLOBAL, int K_GLOBAL)
{
    return workspaceFor(C, tz_workspace_bytes(M_GLOBAL, N_GLOBAL, K_GLOBAL), true);
}

void *sgemmWorkspaceFor(const float *C, int M, int N)
{
    return workspaceFor(C, (long long)M * N * (long long)sizeof(float), false);
}

void tzgemmReleaseWorkspaces()
{
    std::lock_guard<std::mutex> lock(g_workspace_mutex);
    TK_SAFE_CALL(tkDeviceSynchronize());
    for (auto &w : g_workspaces) TK_SAFE_CALL(tkFree(w.second.ptr));
    for (void *p : g_outgrown_workspaces) TK_SAFE_CALL(tkFree(p));
    g_workspaces.clear();
    g_outgrown_workspaces.clear();
    std::fill(g_table_mirror.begin(), g_table_mirror.end(), tz_ws_entry{0, 0});
    TK_SAFE_CALL(tkMemcpyToSymbol("tz_ws_table", g_table_mirror.data(), g_table_mirror.size() * sizeof(tz_ws_entry), 0));
}

static void fmap_insert(const char *key, const void *func, void *)
{
    fmap[key] = const_cast<void *>(func);
}

static bool g_initialised = false;

// tkInit + registry + kinfo; returns a tk error code
int tacker_runtime_init(int device, const char *kinfo_json_path)
{
    if (g_initialised) {
        if (kinfo_json_path && *kinfo_json_path) read_json(kinfo_json_path);
        return TK_SUCCESS;
    }
    int rc = tkInit(device);
    if (rc) return rc;
    rc = tk_register_kernels(fmap_insert, nullptr);
    if (rc) return rc;
    if (kinfo_json_path && *kinfo_json_path) read_json(kinfo_json_path);
    else read_json_text(TK_KINFO_BUILTIN);
    g_initialised = true;
    return TK_SUCCESS;
}

bool tacker_runtime_ready() { return g_initialised; }
