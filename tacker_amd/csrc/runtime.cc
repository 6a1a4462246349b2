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

namespace {
void rebind_workspaces(const void *old_c, const void *new_c);
}

static void grow(void **ptr, long long *have, long long need, bool seed_halves)
{
    if (need <= *have) return;
    TK_SAFE_CALL(tkDeviceSynchronize());   // nothing may still be using the old buffer
    void *old = *ptr;
    if (old) TK_SAFE_CALL(tkFree(old));
    TK_SAFE_CALL(tkMalloc(ptr, (size_t)need));
    if (old && !seed_halves) rebind_workspaces(old, *ptr);   // the output buffer: its workspaces follow it
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
// One workspace per table key (tz_ws_key_tzgemm(C) or tz_ws_key_sgemm(C): the two kinds of kernel
// never share a buffer).  users = kernel objects alive that were built on it; a binding nobody
// uses stays (the next object on the same output buffer finds it) until room is needed.
struct BoundWorkspace {
    void *ptr;
    long long bytes;
    int users;
    unsigned long long last_use;   // value of g_use_clock at the last acquire
    unsigned slot;                 // its slot in the device table
};
constexpr unsigned long long kTombstone = TZ_WS_TOMBSTONE;
std::mutex g_workspace_mutex;
std::unordered_map<unsigned long long, BoundWorkspace> g_workspaces;   // by table key
std::vector<void *> g_outgrown_workspaces;   // replaced by a larger one; launches in flight may still use them
unsigned long long g_use_clock = 0;
constexpr size_t kMaxBoundWorkspaces = TZ_WS_TABLE_SLOTS / 2;   // load factor of the device table
constexpr long long kMaxIdleBytes = 1LL << 30;                  // unused bindings may hold this much device memory
std::vector<tz_ws_entry> g_table_mirror(TZ_WS_TABLE_SLOTS, tz_ws_entry{0, 0});   // host copy of tz_ws_table

void write_slot(unsigned slot, tz_ws_entry e)
{
    g_table_mirror[slot] = e;
    TK_SAFE_CALL(tkMemcpyToSymbol("tz_ws_table", &g_table_mirror[slot], sizeof(tz_ws_entry), slot * sizeof(tz_ws_entry)));
}

// The slot (key, workspace) can go to: the key's own if it has one, else the first empty slot or
// tombstone within the probe window; -1 if the window is full of other keys.  A slot is written
// with one 16-byte copy and a live entry never moves, so a kernel that runs meanwhile and probes
// past it for another key sees it either as it was or whole.
int slot_for(unsigned long long key)
{
    unsigned slot = tz_ws_hash(key);
    int free_slot = -1;
    for (int probe = 0; probe < TZ_WS_TABLE_MAX_PROBES; ++probe, slot = (slot + 1) & (TZ_WS_TABLE_SLOTS - 1)) {
        const unsigned long long c = g_table_mirror[slot].c;
        if (c == key) return (int)slot;
        if (c == 0) return free_slot >= 0 ? free_slot : (int)slot;
        if (c == kTombstone && free_slot < 0) free_slot = (int)slot;
    }
    return free_slot;
}

// Takes a binding out: a tombstone in its slot (the probe chains that pass it stay whole) and the
// buffer freed.  Only after a device synchronisation.
void drop_binding(std::unordered_map<unsigned long long, BoundWorkspace>::iterator it)
{
    write_slot(it->second.slot, tz_ws_entry{kTombstone, 0});
    TK_SAFE_CALL(tkFree(it->second.ptr));
    g_workspaces.erase(it);
}

long long idle_bytes()
{
    long long sum = 0;
    for (auto &w : g_workspaces)
        if (w.second.users == 0) sum += w.second.bytes;
    return sum;
}

// Evicts the least recently used binding without users (among those in the probe window of
// `near_key` when window_only).  The device has been synchronised.  False when there is none.
bool evict_one(unsigned long long near_key, bool window_only)
{
    auto victim = g_workspaces.end();
    const unsigned first = tz_ws_hash(near_key);
    for (auto it = g_workspaces.begin(); it != g_workspaces.end(); ++it) {
        if (it->second.users != 0) continue;
        if (window_only && ((it->second.slot - first) & (TZ_WS_TABLE_SLOTS - 1)) >= TZ_WS_TABLE_MAX_PROBES) continue;
        if (victim == g_workspaces.end() || it->second.last_use < victim->second.last_use) victim = it;
    }
    if (victim == g_workspaces.end()) return false;
    drop_binding(victim);
    return true;
}

// A device buffer of at least `need` bytes bound to `key`, zero when it is new; one more user.
void *acquire_workspace(unsigned long long key, long long need)
{
    std::lock_guard<std::mutex> lock(g_workspace_mutex);
    auto it = g_workspaces.find(key);
    if (it != g_workspaces.end() && it->second.bytes >= need) {
        ++it->second.users;
        it->second.last_use = ++g_use_clock;
        return it->second.ptr;
    }
    // a new binding is rare (first kernel object on this output buffer, or a larger shape), so it may
    // wait for the device -- which also makes this the moment to take out what nobody uses any more
    TK_SAFE_CALL(tkDeviceSynchronize());
    for (void *p : g_outgrown_workspaces) TK_SAFE_CALL(tkFree(p));
    g_outgrown_workspaces.clear();
    while (idle_bytes() > kMaxIdleBytes && evict_one(key, false)) {}
    it = g_workspaces.find(key);   // (the eviction never takes a binding with users, but this one may have none)
    if (it == g_workspaces.end()) {
        while (g_workspaces.size() >= kMaxBoundWorkspaces)
            if (!evict_one(key, false))
                throw std::runtime_error("tzgemm: " + std::to_string(kMaxBoundWorkspaces) +
                                         " output buffers hold a workspace that a live kernel object uses");
        while (slot_for(key) < 0)
            if (!evict_one(key, true))
                throw std::runtime_error("tzgemm: the device table of workspaces has no free slot near this output "
                                         "buffer's hash, and live kernel objects use every binding there");
    }
    void *ptr = nullptr;
    TK_SAFE_CALL(tkMalloc(&ptr, (size_t)need));
    TK_SAFE_CALL(tkMemset(ptr, 0, (size_t)need));
    TK_SAFE_CALL(tkDeviceSynchronize());   // zero before any stream's kernel reads the counters
    const int slot = slot_for(key);
    try {
        write_slot((unsigned)slot, tz_ws_entry{key, (unsigned long long)(size_t)ptr});
    } catch (...) {
        tkErrCheck(tkFree(ptr));
        throw;
    }
    int users = 1;
    if (it != g_workspaces.end()) {
        users += it->second.users;
        g_outgrown_workspaces.push_back(it->second.ptr);
    }
    g_workspaces[key] = BoundWorkspace{ptr, need, users, ++g_use_clock, (unsigned)slot};
    return ptr;
}

void release_workspace(unsigned long long key)
{
    std::lock_guard<std::mutex> lock(g_workspace_mutex);
    auto it = g_workspaces.find(key);
    if (it != g_workspaces.end() && it->second.users > 0) --it->second.users;
}

// The buffer old_c has been freed and new_c takes its place (the global C grew): its bindings
// follow it, so that kernel objects built on the global C keep the workspace they were given,
// and nothing stays bound to an address the allocator may hand out again.  The device has been
// synchronised by the caller.
void rebind_workspaces(const void *old_c, const void *new_c)
{
    std::lock_guard<std::mutex> lock(g_workspace_mutex);
    const unsigned long long keys[2][2] = {{tz_ws_key_tzgemm(old_c), tz_ws_key_tzgemm(new_c)},
                                           {tz_ws_key_sgemm(old_c), tz_ws_key_sgemm(new_c)}};
    for (auto &k : keys) {
        auto it = g_workspaces.find(k[0]);
        if (it == g_workspaces.end()) continue;
        BoundWorkspace w = it->second;
        write_slot(w.slot, tz_ws_entry{kTombstone, 0});
        g_workspaces.erase(it);
        auto stale = g_workspaces.find(k[1]);   // a binding left at the new address by an earlier owner
        if (stale != g_workspaces.end()) {
            w.users += stale->second.users;
            if (stale->second.bytes > w.bytes) std::swap(w.ptr, stale->second.ptr), std::swap(w.bytes, stale->second.bytes);
            drop_binding(stale);
        }
        while (slot_for(k[1]) < 0)
            if (!evict_one(k[1], true)) {
                TK_SAFE_CALL(tkFree(w.ptr));   // the next kernel object built on the buffer binds a new one
                w.ptr = nullptr;
                break;
            }
        if (!w.ptr) continue;
        w.slot = (unsigned)slot_for(k[1]);
        write_slot(w.slot, tz_ws_entry{k[1], (unsigned long long)(size_t)w.ptr});
        g_workspaces[k[1]] = w;
    }
}
}  // namespace

void *tzgemmWorkspaceFor(const float *C, int M_GLOBAL, int N_GLOBAL, int K_GLOBAL)
{
    const long long need = tz_workspace_bytes(M_GLOBAL, N_GLOBAL, K_GLOBAL);
    if (need == 0 || C == nullptr) return nullptr;
    return acquire_workspace(tz_ws_key_tzgemm(C), need);
}

void tzgemmWorkspaceDone(const float *C, int M_GLOBAL, int N_GLOBAL, int K_GLOBAL)
{
    if (tz_workspace_bytes(M_GLOBAL, N_GLOBAL, K_GLOBAL) == 0 || C == nullptr) return;
    release_workspace(tz_ws_key_tzgemm(C));
}

void *sgemmWorkspaceFor(const float *C, int M, int N)
{
    if (C == nullptr) return nullptr;
    return acquire_workspace(tz_ws_key_sgemm(C), (long long)M * N * (long long)sizeof(float));
}

void sgemmWorkspaceDone(const float *C) { if (C) release_workspace(tz_ws_key_sgemm(C)); }

void tzgemmWorkspaceStats(int *bindings, int *in_use, long long *bytes)
{
    std::lock_guard<std::mutex> lock(g_workspace_mutex);
    int used = 0;
    long long sum = 0;
    for (auto &w : g_workspaces) {
        used += w.second.users > 0;
        sum += w.second.bytes;
    }
    if (bindings) *bindings = (int)g_workspaces.size();
    if (in_use) *in_use = used;
    if (bytes) *bytes = sum;
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
