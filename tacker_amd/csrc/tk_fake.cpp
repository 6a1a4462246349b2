// tk_fake.cpp -- recording stand-in for the device layer, for CPU-only tests of
// the host runtime.  "Device" memory is host memory, every launch is appended to
// a log (function key, grid, block, raw bytes of each argument) that tests read
// back through tk_fake_* functions, and nothing is computed.  A launch can be
// made to fail on demand to exercise the error conventions.
#include <cstdlib>
#include <cstring>
#include <map>
#include <string>
#include <vector>

#include "../../include/tacker_amd.h"

namespace {
struct FakeKernel {
    std::string key;
    std::vector<int> arg_sizes;   // bytes of each argument, in order
};
struct Launch {
    std::string key;
    tkDim3 grid, block;
    std::vector<std::vector<unsigned char>> args;
    void *stream;
    bool by_driver = false;   // launched through tkModuleLaunchKernel
};
std::vector<FakeKernel *> &kernels()
{
    static std::vector<FakeKernel *> k;
    return k;
}
std::vector<Launch> g_launches;
// stream capture: launches on the capturing stream are recorded, not "run"; a graph replays its record
void *g_capturing = nullptr;
std::vector<Launch> g_captured;
struct FakeGraph {
    std::vector<Launch> launches;
};
int g_graph_launches = 0;
int g_fail_next_launch = 0;
int g_cu_count = 256;
float g_event_ms = 1.0f;
std::vector<float> g_event_queue;   // scripted durations, consumed first
std::map<std::string, std::vector<unsigned char>> g_symbols;

const int P = 8, I = 4, F = 4;   // pointer, int, float
std::vector<int> trailer(bool with_thread_base)
{
    std::vector<int> t(9, I);
    if (with_thread_base) t.push_back(I);
    return t;
}
std::vector<int> cat(std::vector<int> a, const std::vector<int> &b)
{
    a.insert(a.end(), b.begin(), b.end());
    return a;
}
const std::vector<int> STENCIL = {F, F, P, P, I, I, I};
const std::vector<int> LBM = {P, P};
const std::vector<int> MRIQ = {I, I, P, P, P, P, P};
const std::vector<int> MRIF = {I, I, P, P, P, P, P};
const std::vector<int> CP = {I, F, P};
const std::vector<int> SGEMM = {P, P, P, I, I, I};
const std::vector<int> FFT = {P};
const std::vector<int> NN = {P, P, I, F, F};
const std::vector<int> HOT3D = {P, P, P, F, I, I, I, F, F, F, F, F, F, F};
const std::vector<int> PATH = {I, P, P, P, I, I, I, I};
const std::vector<int> LAVA = {4, 56, P, P, P, P};   // par_str and dim_str by value
const std::vector<int> CUTCP = {I, I, P, F, F, F, P, I};
const std::vector<int> TZ = {P, P, P, I, I, I};
}  // namespace

extern "C" {

int tkInit(int) { return TK_SUCCESS; }
const char *tkGetErrorString(int code)
{
    switch (code) {
        case TK_SUCCESS: return "success";
        case TK_ERROR_INVALID_VALUE: return "invalid value";
        case TK_ERROR_NOT_FOUND: return "not found";
        case TK_ERROR_UNSUPPORTED: return "unsupported shape";
        case TK_ERROR_DEVICE: return "fake device error";
        default: return "unknown error";
    }
}
int tkGetCuCount(int *cu_count) { *cu_count = g_cu_count; return TK_SUCCESS; }
int tkGetDeviceName(char *buf, size_t len) { snprintf(buf, len, "fake device"); return TK_SUCCESS; }
// Allocations come zeroed from calloc without their pages being touched; clearing one that nothing
// has written yet would only touch them (the default instances of the large kernels clear gigabytes).
namespace {
std::map<char *, size_t> g_untouched;   // base -> bytes of allocations still as calloc left them
void touched(void *dst)
{
    auto it = g_untouched.upper_bound(static_cast<char *>(dst));
    if (it == g_untouched.begin()) return;
    --it;
    if (static_cast<char *>(dst) < it->first + it->second) g_untouched.erase(it);
}
}  // namespace
static long long g_malloc_calls = 0, g_free_calls = 0;
int tkAllocationCalls(long long *mallocs, long long *frees)
{
    if (mallocs) *mallocs = g_malloc_calls;
    if (frees) *frees = g_free_calls;
    return TK_SUCCESS;
}
int tkMalloc(void **ptr, size_t bytes)
{
    ++g_malloc_calls;
    *ptr = calloc(1, bytes ? bytes : 1);
    if (!*ptr) return TK_ERROR_DEVICE;
    g_untouched[static_cast<char *>(*ptr)] = bytes ? bytes : 1;
    return TK_SUCCESS;
}
int tkFree(void *ptr)
{
    ++g_free_calls;
    g_untouched.erase(static_cast<char *>(ptr));
    free(ptr);
    return TK_SUCCESS;
}
int tkMemcpy(void *dst, const void *src, size_t bytes, int)
{
    touched(dst);
    memmove(dst, src, bytes);
    return TK_SUCCESS;
}
int tkMemcpyAsync(void *dst, const void *src, size_t bytes, int, tkStream_t)
{
    touched(dst);
    memmove(dst, src, bytes);
    return TK_SUCCESS;
}
int tkMemset(void *ptr, int value, size_t bytes)
{
    auto it = g_untouched.find(static_cast<char *>(ptr));
    if (value == 0 && it != g_untouched.end() && bytes <= it->second) return TK_SUCCESS;   // still all zero
    touched(ptr);
    memset(ptr, value, bytes);
    return TK_SUCCESS;
}
int tkMemcpyToSymbol(const char *symbol, const void *src, size_t bytes, size_t offset)
{
    if (strcmp(symbol, "ck") && strcmp(symbol, "c_mrif") && strcmp(symbol, "atominfo") && strcmp(symbol, "tk_spin_fail") &&
        strcmp(symbol, "tz_ws_table") && strcmp(symbol, "NbrListLen") && strcmp(symbol, "NbrList"))
        return TK_ERROR_NOT_FOUND;
    auto &buf = g_symbols[symbol];
    if (buf.size() < offset + bytes) buf.resize(offset + bytes);
    memcpy(buf.data() + offset, src, bytes);
    return TK_SUCCESS;
}
int tkMemcpyFromSymbol(void *dst, const char *symbol, size_t bytes, size_t offset)
{
    auto it = g_symbols.find(symbol);
    memset(dst, 0, bytes);
    if (it == g_symbols.end()) return strcmp(symbol, "tk_spin_fail") ? TK_ERROR_NOT_FOUND : TK_SUCCESS;
    if (offset + bytes <= it->second.size()) memcpy(dst, it->second.data() + offset, bytes);
    return TK_SUCCESS;
}
int tk_tzgemm_scratch(void **ptr, size_t *bytes)
{
    static std::vector<unsigned char> scratch((8u << 20) + (64u << 10));
    *ptr = scratch.data();
    *bytes = scratch.size();
    return TK_SUCCESS;
}
int tkStreamCreate(tkStream_t *s) { *s = malloc(1); return TK_SUCCESS; }
int tkStreamDestroy(tkStream_t s) { free(s); return TK_SUCCESS; }
int tkStreamSynchronize(tkStream_t) { return TK_SUCCESS; }
int tkDeviceSynchronize(void) { return TK_SUCCESS; }
int tkEventCreate(tkEvent_t *e) { *e = malloc(1); return TK_SUCCESS; }
int tkEventDestroy(tkEvent_t e) { free(e); return TK_SUCCESS; }
int tkEventRecord(tkEvent_t, tkStream_t) { return TK_SUCCESS; }
int tkEventSynchronize(tkEvent_t) { return TK_SUCCESS; }
int tkEventElapsedTime(float *ms, tkEvent_t, tkEvent_t)
{
    if (!g_event_queue.empty()) {
        *ms = g_event_queue.front();
        g_event_queue.erase(g_event_queue.begin());
    } else {
        *ms = g_event_ms;
    }
    return TK_SUCCESS;
}

int tkLaunchKernel(const void *func, tkDim3 grid, tkDim3 block, void **args, size_t, tkStream_t stream)
{
    if (g_fail_next_launch) {
        g_fail_next_launch--;
        return TK_ERROR_DEVICE;
    }
    const FakeKernel *k = nullptr;
    for (auto *cand : kernels())
        if (cand == func) k = cand;
    if (!k) return TK_ERROR_INVALID_VALUE;
    Launch l;
    l.key = k->key;
    l.grid = grid;
    l.block = block;
    l.stream = stream;
    for (size_t i = 0; i < k->arg_sizes.size(); ++i) {
        const unsigned char *p = (const unsigned char *)args[i];
        l.args.emplace_back(p, p + k->arg_sizes[i]);
    }
    if (g_capturing && stream == g_capturing) g_captured.push_back(std::move(l));
    else g_launches.push_back(std::move(l));
    return TK_SUCCESS;
}

int tkStreamBeginCapture(tkStream_t s)
{
    if (!s || g_capturing) return TK_ERROR_INVALID_VALUE;
    g_capturing = s;
    g_captured.clear();
    return TK_SUCCESS;
}
int tkStreamEndCapture(tkStream_t s, tkGraphExec_t *exec)
{
    if (!s || s != g_capturing || !exec) return TK_ERROR_INVALID_VALUE;
    g_capturing = nullptr;
    *exec = new FakeGraph{std::move(g_captured)};
    g_captured.clear();
    return TK_SUCCESS;
}
int tkGraphLaunch(tkGraphExec_t exec, tkStream_t s)
{
    if (!exec) return TK_ERROR_INVALID_VALUE;
    for (Launch l : static_cast<FakeGraph *>(exec)->launches) {
        l.stream = s;
        g_launches.push_back(std::move(l));
    }
    ++g_graph_launches;
    return TK_SUCCESS;
}
int tkGraphExecDestroy(tkGraphExec_t exec)
{
    delete static_cast<FakeGraph *>(exec);
    return TK_SUCCESS;
}

int tkModuleLoad(tkModule_t *m, const char *path)
{
    FILE *f = fopen(path, "rb");
    if (!f) return TK_ERROR_DEVICE;
    fclose(f);
    *m = malloc(1);
    return TK_SUCCESS;
}
int tkModuleUnload(tkModule_t m) { free(m); return TK_SUCCESS; }
// a fake code object holds every kernel of the registry, under the name its device function has in
// the real one: general_ptb_<kernel> (g_general_ptb_<kernel> for mriq and cp) for gptb_<kernel>
int tkModuleGetFunction(tkFunction_t *f, tkModule_t, const char *name)
{
    std::string key = name;
    for (const char *prefix : {"g_general_ptb_", "general_ptb_"})
        if (key.rfind(prefix, 0) == 0) {
            key = "gptb_" + key.substr(strlen(prefix));
            break;
        }
    for (auto *k : kernels())
        if (k->key == key) { *f = k; return TK_SUCCESS; }
    return TK_ERROR_NOT_FOUND;
}
int tkModuleLaunchKernel(tkFunction_t f, tkDim3 grid, tkDim3 block, void **args, size_t shmem, tkStream_t s)
{
    const int rc = tkLaunchKernel(f, grid, block, args, shmem, s);
    if (rc == TK_SUCCESS) g_launches.back().by_driver = true;
    return rc;
}

int tk_register_kernels(tk_kernel_insert_fn insert, void *ctx)
{
    if (kernels().empty()) {
        auto add = [](const std::string &key, std::vector<int> sizes) {
            kernels().push_back(new FakeKernel{key, std::move(sizes)});
        };
        add("ori_stencil", STENCIL);
        add("ori_lbm", LBM);
        add("ori_ComputePhiMag", {P, P, P, I});
        add("ori_mriq", MRIQ);
        add("ori_cp", CP);
        add("ComputeRhoPhiGPU", {I, P, P, P, P, P, P});
        add("ori_mrif", MRIF);
        add("ori_sgemm", SGEMM);
        add("ori_fft", FFT);
        add("ori_cutcp", CUTCP);
        add("ori_nn", NN);
        add("ori_hot3d", HOT3D);
        add("ori_path", PATH);
        add("ori_lava", LAVA);
        add("fill_uniform", {P, 8, I, F, F});
        add("fill_int_mod", {P, 8, I, I});
        add("gptb_tzgemm", cat(TZ, trailer(true)));
        add("gptb_tzgemm@large", cat(TZ, trailer(true)));
        add("gptb_tzgemm_scratch", cat(cat(TZ, {P}), trailer(true)));
        add("tz_clear_words", {P, I});
        add("gptb_stencil", cat(STENCIL, trailer(true)));
        add("gptb_lbm", cat(LBM, trailer(true)));
        add("gptb_mriq", cat(MRIQ, trailer(true)));
        add("gptb_cp", cat(CP, trailer(true)));
        add("gptb_mrif", cat(MRIF, trailer(true)));
        add("gptb_sgemm", cat(SGEMM, trailer(true)));
        add("gptb_fft", cat(FFT, trailer(true)));
        add("gptb_cutcp", cat(CUTCP, trailer(true)));
        add("gptb_nn", cat(NN, trailer(true)));
        add("gptb_hot3d", cat(HOT3D, trailer(true)));
        add("gptb_path", cat(PATH, trailer(true)));
        add("gptb_lava", cat(LAVA, trailer(true)));
        add("cp_inv_sqrt_selftest", {I, I, P});
        add("im2col", {I, P, I, I, I, I, I, I, I, I, I, I, I, I, P, I, I});
        add("convert_fp32_to_fp16", {P, P, I});
        add("im2col_nhwc_f16", {P, I, I, I, I, I, I, I, I, I, I, P, I, P, I, I});
        add("im2col3x3_scatter_nhwc_f16", {P, I, I, I, I, P, I, P, I, I});
        add("maxpool2x2_nhwc", {P, I, I, I, P, P, I});
        add("pack_fc_input", {P, 8, P, I, I, P});
        add("pack_fc_input_pooled", {P, I, I, I, P, I, I, P});
        const std::pair<const char *, const std::vector<int> *> bes[] = {
            {"stencil", &STENCIL}, {"lbm", &LBM}, {"mriq", &MRIQ}, {"cp", &CP}, {"mrif", &MRIF}, {"sgemm", &SGEMM},
            {"fft", &FFT}, {"cutcp", &CUTCP}};
        static const char *variants[] = {"", "@wg_1_1", "@wg_1_2", "@wave_256", "@wave_512"};
        // the Rodinia kernels pair with tzgemm and with each other only
        const std::pair<const char *, const std::vector<int> *> rodinia[] = {{"nn", &NN}, {"hot3d", &HOT3D}, {"path", &PATH}, {"lava", &LAVA}};
        for (auto *family : {&bes[0], &rodinia[0]})
            for (auto *be = family; be != family + (family == &bes[0] ? 8 : 4); ++be)
                for (auto v : variants)
                    add((std::string("tzgemm_") + be->first + v).c_str(),
                        cat(cat(*be->second, trailer(false)), cat(TZ, trailer(false))));
        // best-effort pairs, first < second alphabetically
        static const char *pair_variants[] = {"", "@wg_1_1", "@wg_1_2", "@wg_2_1", "@ord_1_1", "@ord_1_2", "@ord_2_1"};
        for (auto *family : {&bes[0], &rodinia[0]}) {
            const int n = family == &bes[0] ? 8 : 4;
            for (auto *a = family; a != family + n; ++a)
                for (auto *b = family; b != family + n; ++b)
                    if (std::string(a->first) < std::string(b->first))
                        for (auto v : pair_variants)
                            add((std::string(a->first) + "_" + b->first + v).c_str(),
                                cat(cat(*a->second, trailer(false)), cat(*b->second, trailer(false))));
        }
    }
    for (auto *k : kernels()) insert(k->key.c_str(), k, ctx);
    return TK_SUCCESS;
}

// ---- inspection interface for tests --------------------------------------
TK_API int tk_fake_launch_count(void) { return (int)g_launches.size(); }
TK_API int tk_fake_graph_launch_count(void) { return g_graph_launches; }
TK_API void tk_fake_reset(void) { g_launches.clear(); g_graph_launches = 0; g_fail_next_launch = 0; g_event_queue.clear(); }
TK_API void tk_fake_fail_next_launches(int n) { g_fail_next_launch = n; }
TK_API void tk_fake_set_cu_count(int n) { g_cu_count = n; }
TK_API void tk_fake_set_event_ms(float ms) { g_event_ms = ms; }
TK_API void tk_fake_push_event_ms(const float *ms, int n) { g_event_queue.insert(g_event_queue.end(), ms, ms + n); }
TK_API int tk_fake_event_queue_len(void) { return (int)g_event_queue.size(); }
TK_API const char *tk_fake_launch_key(int i) { return g_launches[i].key.c_str(); }
TK_API int tk_fake_launch_by_driver(int i) { return g_launches[i].by_driver ? 1 : 0; }
TK_API int tk_fake_launch_nargs(int i) { return (int)g_launches[i].args.size(); }
TK_API void tk_fake_launch_dims(int i, unsigned out[6])
{
    const Launch &l = g_launches[i];
    out[0] = l.grid.x; out[1] = l.grid.y; out[2] = l.grid.z;
    out[3] = l.block.x; out[4] = l.block.y; out[5] = l.block.z;
}
// copies argument a of launch i into out (up to cap bytes), returns its size
TK_API int tk_fake_launch_arg(int i, int a, void *out, int cap)
{
    const auto &v = g_launches[i].args[a];
    memcpy(out, v.data(), (size_t)cap < v.size() ? (size_t)cap : v.size());
    return (int)v.size();
}
TK_API int tk_fake_symbol(const char *name, void *out, int cap)
{
    auto it = g_symbols.find(name);
    if (it == g_symbols.end()) return -1;
    memcpy(out, it->second.data(), (size_t)cap < it->second.size() ? (size_t)cap : it->second.size());
    return (int)it->second.size();
}

}  // extern "C"
