// capi.cc -- the tacker_* entry points of include/tacker_amd.h.
// Each one validates its arguments (returning a code instead of letting the
// class layer's logger.ERROR end the process), then builds and runs the same
// Kernel / GPTBKernel / MixKernel objects a C++ caller would.
#include <cstring>
#include <memory>
#include <stdexcept>
#include <string>

#include "Creator.h"
#include "Logger.h"
#include "json.h"
#include "rng.h"
#include "TaskManager.h"
#include "dnn/vgg16.h"
#include "header/stencil_header.h"

extern Logger logger;
extern std::unordered_map<std::string, void *> fmap;
int tacker_runtime_init(int device, const char *kinfo_json_path);
extern "C" int tk_tzgemm_scratch(void **ptr, size_t *bytes);   // beside the array, in the device translation unit
bool tacker_runtime_ready();

namespace {
thread_local std::string g_error;

int fail(int code, const std::string &msg)
{
    g_error = msg;
    return code;
}

// run f(), mapping exceptions of the class layer to an error code
template <class F>
int guarded(F &&f)
{
    try {
        return f();
    } catch (const std::exception &e) {
        return fail(TK_ERROR_DEVICE, e.what());
    }
}

#define REQUIRE_INIT()                                                             \
    do {                                                                           \
        if (!tacker_runtime_ready()) return fail(TK_ERROR_INVALID_VALUE, "tacker_init has not been called"); \
    } while (0)

bool has_key(const std::string &key) { return fmap.find(key) != fmap.end(); }

// Creator geometry of the plain GPTB launch of a kernel on this GPU
int default_block(const std::string &name)
{
    const int bs = get_kernel_info(name, "blocksize");
    return bs == JSON_NOT_FOUND ? 256 : bs;
}
int default_grid(const std::string &name)
{
    int per_cu = get_kernel_info(name, "solo_ptb_blks");
    if (per_cu == JSON_NOT_FOUND || per_cu < 1) per_cu = 1;
    return cuCount() * per_cu;
}

int check_block(const std::string &name, int block)
{
    if (block <= 0 || block % 64 || block > 256)
        return fail(TK_ERROR_INVALID_VALUE, name + ": launch_block must be a multiple of 64 in [64,256]");
    if (name == "tzgemm" && block != TZ_THREADS)
        return fail(TK_ERROR_INVALID_VALUE, "tzgemm: launch_block must be 256");
    if ((name == "mriq" || name == "mrif") && block % 256)
        return fail(TK_ERROR_INVALID_VALUE, name + ": launch_block must be a multiple of 256");
    if ((name == "cp" || name == "sgemm") && block % 128)
        return fail(TK_ERROR_INVALID_VALUE, name + ": launch_block must be a multiple of 128");
    return TK_SUCCESS;
}

GPTBKernel *make_gptb(Kernel *ori, int launch_grid, int launch_block, int start, int end)
{
    const std::string &name = ori->kernelName;
    const int grid = launch_grid > 0 ? launch_grid : default_grid(name);
    const int block = launch_block > 0 ? launch_block : default_block(name);
    return new GPTBKernel(ori->Id, name, "gptb_" + name, ori, dim3(grid, 1, 1), dim3(block, 1, 1), start, end);
}

int natural_blocks(Kernel *ori)
{
    return (int)(ori->launchGridDim.x * ori->launchGridDim.y * ori->launchGridDim.z);
}

int check_range(Kernel *ori, int start, int end)
{
    if (start < 0 || end < start) return fail(TK_ERROR_INVALID_VALUE, ori->kernelName + ": bad block range");
    if (ori->kernelName == "tzgemm" && end > natural_blocks(ori))
        return fail(TK_ERROR_INVALID_VALUE, "tzgemm: tile range exceeds the tile count");
    return TK_SUCCESS;
}

int check_stencil(const float *A0, float *Anext, int nx, int ny, int nz)
{
    if (!A0 || !Anext || nx < 1 || ny < 1 || nz < 1) return fail(TK_ERROR_INVALID_VALUE, "stencil: bad arguments");
    if ((long long)nx * ny * nz >= (1LL << 40)) return fail(TK_ERROR_UNSUPPORTED, "stencil: grid too large");
    return TK_SUCCESS;
}
int check_lbm(const float *src, float *dst, int sx, int sy, int sz)
{
    if (!src || !dst || sx < 1 || sy < 1 || sz < 1) return fail(TK_ERROR_INVALID_VALUE, "lbm: bad arguments");
    if ((long long)sx * sy * sz * 20 >= (1LL << 31)) return fail(TK_ERROR_UNSUPPORTED, "lbm: grid too large for 32-bit cell indices");
    return TK_SUCCESS;
}
int check_mriq(int numK, const float *x, const float *y, const float *z, float *Qr, float *Qi, int numX)
{
    if (!x || !y || !z || !Qr || !Qi || numK < 0 || numK > MRIQ_MAX_K || numX < 0)
        return fail(TK_ERROR_INVALID_VALUE, "mriq: bad arguments");
    if (numX % KERNEL_Q_THREADS_PER_BLOCK) return fail(TK_ERROR_UNSUPPORTED, "mriq: numX must be a multiple of 256");
    return TK_SUCCESS;
}
int check_mrif(int numK, const float *x, const float *y, const float *z, float *outR, float *outI, int numX)
{
    if (!x || !y || !z || !outR || !outI || numK < 0 || numK > MRIF_MAX_K || numX < 0)
        return fail(TK_ERROR_INVALID_VALUE, "mrif: bad arguments");
    if (numX % KERNEL_FH_THREADS_PER_BLOCK) return fail(TK_ERROR_UNSUPPORTED, "mrif: numX must be a multiple of 256");
    return TK_SUCCESS;
}
int check_cp(int numatoms, float *grid, int volx, int voly)
{
    if (!grid || numatoms < 0 || numatoms > MAXATOMS) return fail(TK_ERROR_INVALID_VALUE, "cp: bad arguments");
    if (volx < 128 || voly < 8 || volx % (BLOCKSIZEX * UNROLLX) || voly % BLOCKSIZEY)
        return fail(TK_ERROR_UNSUPPORTED, "cp: volx must be a multiple of 128 and voly of 8");
    return TK_SUCCESS;
}
int check_gemm(const void *A, const void *B, float *C, int M, int N, int K)
{
    if (!A || !B || !C) return fail(TK_ERROR_INVALID_VALUE, "tzgemm: null operand");
    if (M < 128 || N < 128 || K < 128 || M % 128 || N % 128 || K % 128)
        return fail(TK_ERROR_UNSUPPORTED, "tzgemm: M, N, K must be multiples of 128");
    return TK_SUCCESS;
}

// launch an ori object once and drop it
int run_once(Kernel *k, tkStream_t stream)
{
    std::unique_ptr<Kernel> hold(k);
    return guarded([&]() -> int {
        k->execute(stream);
        return TK_SUCCESS;
    });
}
int run_gptb_once(Kernel *ori, int start, int end, int grid, int block, tkStream_t stream)
{
    std::unique_ptr<Kernel> hold_ori(ori);
    int rc = check_range(ori, start, end);
    if (rc) return rc;
    rc = check_block(ori->kernelName, block > 0 ? block : default_block(ori->kernelName));
    if (rc) return rc;
    return guarded([&]() -> int {
        std::unique_ptr<GPTBKernel> g(make_gptb(ori, grid, block, start, end));
        g->execute(stream);
        return TK_SUCCESS;
    });
}
int run_mix_once(Kernel *be_ori, int be_start, int be_end, const void *A, const void *B, float *C, int M,
                 int N, int K, int tile_start, int tile_end, const char *variant, int grid, int block,
                 tkStream_t stream)
{
    std::unique_ptr<Kernel> hold_be(be_ori);
    int rc = check_gemm(A, B, C, M, N, K);
    if (rc) return rc;
    rc = check_range(be_ori, be_start, be_end);
    if (rc) return rc;
    const std::string v = variant ? variant : "";
    const std::string key = "tzgemm_" + be_ori->kernelName + (v.empty() ? "" : "@" + v);
    if (!has_key(key)) return fail(TK_ERROR_NOT_FOUND, "no fused kernel {" + key + "}");
    if (get_kernel_info(key, "blocksize") == JSON_NOT_FOUND) return fail(TK_ERROR_NOT_FOUND, "kinfo has no entry for {" + key + "}");
    if (block > 0 && block != get_kernel_info(key, "blocksize"))
        return fail(TK_ERROR_INVALID_VALUE, "{" + key + "} is built for " + std::to_string(get_kernel_info(key, "blocksize")) + " threads");
    return guarded([&]() -> int {
        std::unique_ptr<OriTZGEMMKernel> tz_ori(new OriTZGEMMKernel(0, M, N, K, A, B, C));
        int rc2 = check_range(tz_ori.get(), tile_start, tile_end);
        if (rc2) return rc2;
        std::unique_ptr<GPTBKernel> be(make_gptb(be_ori, 0, 0, be_start, be_end));
        std::unique_ptr<GPTBKernel> tz(make_gptb(tz_ori.get(), 0, TZ_THREADS, tile_start, tile_end));
        std::unique_ptr<MixKernel> mix(createTzgemmMix(be.get(), tz.get(), be_start, be_end, tile_start, tile_end, v, grid, block));
        mix->execute(stream);
        return TK_SUCCESS;
    });
}
}  // namespace

extern "C" {

int tacker_init(int device, const char *kinfo_json_path)
{
    return guarded([&]() -> int {
        const int rc = tacker_runtime_init(device, kinfo_json_path);
        if (rc) g_error = tkGetErrorString(rc);
        return rc;
    });
}

const char *tacker_last_error(void) { return g_error.c_str(); }

int tacker_tzgemm_grid_dim(int m, int n, int k, int out[4])
{
    const std::vector<int> d = getTZGEMMGridDim(m, n, k);
    for (int i = 0; i < 4; ++i) out[i] = d[i];
    return TK_SUCCESS;
}

int tacker_tzgemm_parts(int m, int n, int k)
{
    const std::vector<int> d = getTZGEMMGridDim(m, n, k);
    return tz_ksplit_parts(d[0], d[1], d[2]);
}

long long tacker_tzgemm_workspace_bytes(int m, int n, int k)
{
    const std::vector<int> d = getTZGEMMGridDim(m, n, k);
    return tz_workspace_bytes(d[0], d[1], d[2]);
}

int tacker_tzgemm_release_workspaces(void)
{
    REQUIRE_INIT();
    return guarded([&]() -> int {
        tzgemmReleaseWorkspaces();
        return TK_SUCCESS;
    });
}

int tacker_tzgemm_workspace_stats(int *bindings, int *in_use, long long *bytes)
{
    tzgemmWorkspaceStats(bindings, in_use, bytes);
    return TK_SUCCESS;
}

int tacker_global_gemm_buffers(const void **A, const void **B, float **C, long long bytes[3])
{
    if (!A || !B || !C || !bytes) return fail(TK_ERROR_INVALID_VALUE, "null output");
    *A = ori_wmma_A;
    *B = ori_wmma_B;
    *C = ori_wmma_C;
    bytes[0] = MAX_ORI_WMMA_A;
    bytes[1] = MAX_ORI_WMMA_B;
    bytes[2] = MAX_ORI_WMMA_C;
    return TK_SUCCESS;
}

int tacker_gptb_tzgemm(const void *A, const void *B, float *C, int M, int N, int K, int tile_start,
                       int tile_end, int launch_grid, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_gemm(A, B, C, M, N, K);
    if (rc) return rc;
    Kernel *ori = nullptr;   // binding a workspace to C can fail (allocation): not outside guarded()
    const int made = guarded([&]() -> int {
        ori = new OriTZGEMMKernel(0, M, N, K, A, B, C);
        return TK_SUCCESS;
    });
    if (made) return made;
    return run_gptb_once(ori, tile_start, tile_end, launch_grid, TZ_THREADS, stream);
}

int tacker_gptb_tzgemm_static_scratch(const void *A, const void *B, float *C, int M, int N, int K, int tile_start,
                                      int tile_end, int launch_grid, tkStream_t stream)
{
    static_assert(TACKER_TZGEMM_STATIC_SCRATCH_BYTES == TZ_SCRATCH_BYTES, "public and device array sizes must agree");
    REQUIRE_INIT();
    const int rc = check_gemm(A, B, C, M, N, K);
    if (rc) return rc;
    const int tiles = (M / TZ_REF_TILE) * (N / TZ_REF_TILE);
    if (tile_start < 0 || tile_end < tile_start || tile_end > tiles)
        return fail(TK_ERROR_INVALID_VALUE, "tzgemm: bad tile range");
    void *scratch = nullptr;
    size_t scratch_bytes = 0;
    if (tk_tzgemm_scratch(&scratch, &scratch_bytes) != TK_SUCCESS)
        return fail(TK_ERROR_INVALID_VALUE, "tzgemm: the current device's static scratch array was never set up (tacker_init)");
    const long long need = tz_workspace_bytes(M, N, K);
    if (need > (long long)scratch_bytes)
        return fail(TK_ERROR_UNSUPPORTED, "tzgemm: this shape needs a workspace of " + std::to_string(need) +
                                              " bytes, the static scratch array holds " + std::to_string(scratch_bytes));
    auto clear = fmap.find("tz_clear_words");
    auto gemm = fmap.find("gptb_tzgemm_scratch");
    auto large = fmap.find("gptb_tzgemm@large");
    if (clear == fmap.end() || gemm == fmap.end() || large == fmap.end())
        return fail(TK_ERROR_NOT_FOUND, "no kernel {gptb_tzgemm_scratch}");
    if (need > 0) {
        // every call on this GPU shares the array and it keeps the last call's contents: the
        // arrival counters of this shape must start at zero
        int words = (int)(tz_workspace_counter_bytes(M, N) / 4);
        void *clear_args[] = {&scratch, &words};
        const int rc2 = tkLaunchKernel(clear->second, dim3((words + 255) / 256).raw(), dim3(256).raw(), clear_args, 0, stream);
        if (rc2) return fail(rc2, tkGetErrorString(rc2));
    }
    int grid = launch_grid > 0 ? launch_grid : default_grid("tzgemm");
    int dims[6] = {tiles, 1, 1, TZ_THREADS, 1, 1};
    int thread_base = 0;
    void *workspace = need > 0 ? scratch : nullptr;
    void *args[] = {&A, &B, &C, &M, &N, &K, &workspace, &dims[0], &dims[1], &dims[2], &dims[3], &dims[4], &dims[5],
                    &tile_start, &grid, &tile_end, &thread_base};
    int rc3;
    if (tz_use_large(M, N, K)) {
        // the large-tile build takes general_ptb_tzgemm's list (it never needs a workspace)
        void *largs[] = {&A, &B, &C, &M, &N, &K, &dims[0], &dims[1], &dims[2], &dims[3], &dims[4], &dims[5],
                         &tile_start, &grid, &tile_end, &thread_base};
        rc3 = tkLaunchKernel(large->second, dim3(grid).raw(), dim3(TZ_THREADS).raw(), largs, 0, stream);
    } else {
        rc3 = tkLaunchKernel(gemm->second, dim3(grid).raw(), dim3(TZ_THREADS).raw(), args, 0, stream);
    }
    return rc3 ? fail(rc3, tkGetErrorString(rc3)) : rc3;
}

int tacker_ori_stencil(float c0, float c1, const float *A0, float *Anext, int nx, int ny, int nz, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_stencil(A0, Anext, nx, ny, nz);
    if (rc) return rc;
    return run_once(new OriSTENCILKernel(0, c0, c1, A0, Anext, nx, ny, nz), stream);
}

int tacker_stencil_blocks(int nx, int ny, int nz)
{
    static_assert(TACKER_STENCIL_Z_RUN == STENCIL_Z_RUN, "public and device run lengths must agree");
    if (nx < 1 || ny < 1 || nz < 1) return 0;
    const int runs = nz > 2 ? (nz - 2 + STENCIL_Z_RUN - 1) / STENCIL_Z_RUN : 1;
    return ((nx + STENCIL_TILE_X * 2 - 1) / (STENCIL_TILE_X * 2)) * ((ny + STENCIL_TILE_Y - 1) / STENCIL_TILE_Y) * runs;
}

int tacker_gptb_stencil(float c0, float c1, const float *A0, float *Anext, int nx, int ny, int nz,
                        int block_start, int block_end, int launch_grid, int launch_block, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_stencil(A0, Anext, nx, ny, nz);
    if (rc) return rc;
    return run_gptb_once(new OriSTENCILKernel(0, c0, c1, A0, Anext, nx, ny, nz), block_start, block_end,
                         launch_grid, launch_block, stream);
}

int tacker_ori_lbm(const float *src, float *dst, int sx, int sy, int sz, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_lbm(src, dst, sx, sy, sz);
    if (rc) return rc;
    if (sx > 1024) return fail(TK_ERROR_UNSUPPORTED, "ori_lbm: sx above 1024 needs the GPTB form");
    return run_once(new OriLBMKernel(0, src, dst, sx, sy, sz), stream);
}

int tacker_gptb_lbm(const float *src, float *dst, int sx, int sy, int sz, int block_start, int block_end,
                    int launch_grid, int launch_block, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_lbm(src, dst, sx, sy, sz);
    if (rc) return rc;
    return run_gptb_once(new OriLBMKernel(0, src, dst, sx, sy, sz), block_start, block_end, launch_grid,
                         launch_block, stream);
}

int tacker_mriq_phimag(const float *phiR, const float *phiI, float *phiMag, int numK, tkStream_t stream)
{
    REQUIRE_INIT();
    if (!phiR || !phiI || !phiMag || numK < 0) return fail(TK_ERROR_INVALID_VALUE, "mriq_phimag: bad arguments");
    if (numK == 0) return TK_SUCCESS;
    void *args[] = {&phiR, &phiI, &phiMag, &numK};
    const dim3 grid((numK + KERNEL_PHI_MAG_THREADS_PER_BLOCK - 1) / KERNEL_PHI_MAG_THREADS_PER_BLOCK);
    const int rc = tkLaunchKernel(fmap["ori_ComputePhiMag"], grid.raw(), dim3(KERNEL_PHI_MAG_THREADS_PER_BLOCK).raw(), args, 0, stream);
    return rc ? fail(rc, tkGetErrorString(rc)) : rc;
}

int tacker_mriq_set_kvalues(const float *kvals_host, int numK)
{
    REQUIRE_INIT();
    if (!kvals_host || numK < 0 || numK > MRIQ_MAX_K) return fail(TK_ERROR_INVALID_VALUE, "mriq: numK out of range");
    const int rc = OriMRIQKernel::setKValues(reinterpret_cast<const mriq_kValues *>(kvals_host), numK);
    return rc ? fail(rc, tkGetErrorString(rc)) : rc;
}

int tacker_mriq_blocks(int numK, int numX)
{
    static_assert(TACKER_MRIQ_K_CHUNK == MRIQ_K_CHUNK, "public and device chunk sizes must agree");
    if (numK < 0 || numX < 0) return 0;
    const int chunks = numK > 0 ? (numK + MRIQ_K_CHUNK - 1) / MRIQ_K_CHUNK : 1;
    return (numX / KERNEL_Q_THREADS_PER_BLOCK) * chunks;
}

int tacker_ori_mriq(int numK, const float *x, const float *y, const float *z, float *Qr, float *Qi, int numX, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_mriq(numK, x, y, z, Qr, Qi, numX);
    if (rc) return rc;
    if (numX == 0) return TK_SUCCESS;
    return run_once(new OriMRIQKernel(0, numK, x, y, z, Qr, Qi, numX), stream);
}

int tacker_gptb_mriq(int numK, const float *x, const float *y, const float *z, float *Qr, float *Qi, int numX,
                     int block_start, int block_end, int launch_grid, int launch_block, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_mriq(numK, x, y, z, Qr, Qi, numX);
    if (rc) return rc;
    if (numX == 0) return TK_SUCCESS;
    return run_gptb_once(new OriMRIQKernel(0, numK, x, y, z, Qr, Qi, numX), block_start, block_end, launch_grid,
                         launch_block, stream);
}

int tacker_mrif_rhophi(int numK, const float *phiR, const float *phiI, const float *dR, const float *dI,
                       float *realRhoPhi, float *imagRhoPhi, tkStream_t stream)
{
    REQUIRE_INIT();
    if (!phiR || !phiI || !dR || !dI || !realRhoPhi || !imagRhoPhi || numK < 0)
        return fail(TK_ERROR_INVALID_VALUE, "mrif_rhophi: bad arguments");
    if (numK == 0) return TK_SUCCESS;
    void *args[] = {&numK, &phiR, &phiI, &dR, &dI, &realRhoPhi, &imagRhoPhi};
    const dim3 grid((numK + KERNEL_RHO_PHI_THREADS_PER_BLOCK - 1) / KERNEL_RHO_PHI_THREADS_PER_BLOCK);
    const int rc = tkLaunchKernel(fmap["ComputeRhoPhiGPU"], grid.raw(), dim3(KERNEL_RHO_PHI_THREADS_PER_BLOCK).raw(), args, 0, stream);
    return rc ? fail(rc, tkGetErrorString(rc)) : rc;
}

int tacker_mrif_set_kvalues(const float *kvals_host, int numK)
{
    REQUIRE_INIT();
    if (!kvals_host || numK < 0 || numK > MRIF_MAX_K) return fail(TK_ERROR_INVALID_VALUE, "mrif: numK out of range");
    const int rc = OriMRIFKernel::setKValues(reinterpret_cast<const mrif_kValues *>(kvals_host), numK);
    return rc ? fail(rc, tkGetErrorString(rc)) : rc;
}

int tacker_mrif_blocks(int numK, int numX)
{
    static_assert(TACKER_MRIF_K_CHUNK == MRIF_K_CHUNK, "public and device chunk sizes must agree");
    if (numK < 0 || numX < 0) return 0;
    const int chunks = numK > 0 ? (numK + MRIF_K_CHUNK - 1) / MRIF_K_CHUNK : 1;
    return (numX / KERNEL_FH_THREADS_PER_BLOCK) * chunks;
}

int tacker_ori_mrif(int numK, const float *x, const float *y, const float *z, float *outR, float *outI, int numX, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_mrif(numK, x, y, z, outR, outI, numX);
    if (rc) return rc;
    if (numX == 0) return TK_SUCCESS;
    return run_once(new OriMRIFKernel(0, numK, x, y, z, outR, outI, numX), stream);
}

int tacker_gptb_mrif(int numK, const float *x, const float *y, const float *z, float *outR, float *outI, int numX,
                     int block_start, int block_end, int launch_grid, int launch_block, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_mrif(numK, x, y, z, outR, outI, numX);
    if (rc) return rc;
    if (numX == 0) return TK_SUCCESS;
    return run_gptb_once(new OriMRIFKernel(0, numK, x, y, z, outR, outI, numX), block_start, block_end, launch_grid,
                         launch_block, stream);
}

namespace {
int check_sgemm(const float *A, const float *B, float *C, int M, int N, int K)
{
    if (!A || !B || !C || M <= 0 || N <= 0 || K <= 0) return fail(TK_ERROR_INVALID_VALUE, "sgemm: bad arguments");
    if (M % SGEMM_TILE_M || N % SGEMM_TILE_N)
        return fail(TK_ERROR_UNSUPPORTED, "sgemm: M must be a multiple of 128 and N of 16");
    if ((long long)M * K >= (1ll << 31) || (long long)N * K >= (1ll << 31) || (long long)M * N >= (1ll << 31))
        return fail(TK_ERROR_UNSUPPORTED, "sgemm: a matrix of 2^31 elements or more");
    return TK_SUCCESS;
}
}  // namespace

int tacker_sgemm_blocks(int M, int N, int K)
{
    static_assert(TACKER_SGEMM_K_CHUNK == SGEMM_K_CHUNK, "public and device chunk sizes must agree");
    if (M < 0 || N < 0 || K <= 0) return 0;
    return (M / SGEMM_TILE_M) * (N / SGEMM_TILE_N) * ((K + SGEMM_K_CHUNK - 1) / SGEMM_K_CHUNK);
}

int tacker_ori_sgemm(const float *A, const float *B, float *C, int M, int N, int K, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_sgemm(A, B, C, M, N, K);
    if (rc) return rc;
    Kernel *ori = nullptr;   // binding a workspace to C can fail (allocation): not outside guarded()
    const int made = guarded([&]() -> int {
        ori = new OriSGEMMKernel(0, A, B, C, M, N, K);
        return TK_SUCCESS;
    });
    if (made) return made;
    return run_once(ori, stream);
}

int tacker_gptb_sgemm(const float *A, const float *B, float *C, int M, int N, int K, int block_start, int block_end,
                      int launch_grid, int launch_block, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_sgemm(A, B, C, M, N, K);
    if (rc) return rc;
    Kernel *ori = nullptr;
    const int made = guarded([&]() -> int {
        ori = new OriSGEMMKernel(0, A, B, C, M, N, K);
        return TK_SUCCESS;
    });
    if (made) return made;
    return run_gptb_once(ori, block_start, block_end, launch_grid, launch_block, stream);
}

namespace {
int check_fft(const float *data, int batches)
{
    static_assert(TACKER_FFT_POINTS == FFT_N, "public and device transform sizes must agree");
    if (!data || batches <= 0) return fail(TK_ERROR_INVALID_VALUE, "fft: bad arguments");
    if ((long long)batches * FFT_N >= (1ll << 30)) return fail(TK_ERROR_UNSUPPORTED, "fft: a batch of 2^30 points or more");
    return TK_SUCCESS;
}
}  // namespace

int tacker_ori_fft(float *data, int batches, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_fft(data, batches);
    if (rc) return rc;
    return run_once(new OriFFTKernel(0, data, batches), stream);
}

int tacker_gptb_fft(float *data, int batches, int block_start, int block_end, int launch_grid, int launch_block,
                    tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_fft(data, batches);
    if (rc) return rc;
    return run_gptb_once(new OriFFTKernel(0, data, batches), block_start, block_end, launch_grid, launch_block, stream);
}

namespace {
int check_nn(const float *locations, float *distances, int numRecords)
{
    if (!locations || !distances || numRecords <= 0) return fail(TK_ERROR_INVALID_VALUE, "nn: bad arguments");
    return TK_SUCCESS;
}
int check_hot3d(const float *p, const float *tIn, float *tOut, int nx, int ny, int nz)
{
    if (!p || !tIn || !tOut || nx <= 0 || ny <= 0 || nz <= 0 || tIn == tOut)
        return fail(TK_ERROR_INVALID_VALUE, "hot3d: bad arguments");
    if (nx % HOT3D_TILE_X || ny % HOT3D_TILE_Y || nz < 2)
        return fail(TK_ERROR_UNSUPPORTED, "hot3d: nx must be a multiple of 64, ny of 4, and nz at least 2");
    if ((long long)nx * ny * nz >= (1ll << 31)) return fail(TK_ERROR_UNSUPPORTED, "hot3d: a chip of 2^31 cells or more");
    return TK_SUCCESS;
}
int check_path(int iteration, const int *wall, const int *src, int *results, int cols, int rows, int startStep)
{
    if (!wall || !src || !results || cols <= 0 || rows <= 0 || startStep < 0 || src == results)
        return fail(TK_ERROR_INVALID_VALUE, "path: bad arguments");
    if (iteration < 1 || 2 * iteration * PATH_HALO >= PATH_BLOCK_SIZE)
        return fail(TK_ERROR_UNSUPPORTED, "path: a pyramid of 1 .. 127 rows");
    if ((long long)startStep + iteration > rows - 1)
        return fail(TK_ERROR_INVALID_VALUE, "path: the pyramid reaches past the wall's last row");
    if ((long long)cols * rows >= (1ll << 31)) return fail(TK_ERROR_UNSUPPORTED, "path: a wall of 2^31 cells or more");
    return TK_SUCCESS;
}
}  // namespace

int tacker_nn_blocks(int numRecords) { return nnBlocks(numRecords); }

int tacker_ori_nn(const float *locations, float *distances, int numRecords, float lat, float lng, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_nn(locations, distances, numRecords);
    if (rc) return rc;
    return run_once(new OriNNKernel(0, (LatLong *)const_cast<float *>(locations), distances, numRecords, lat, lng), stream);
}

int tacker_gptb_nn(const float *locations, float *distances, int numRecords, float lat, float lng, int block_start,
                   int block_end, int launch_grid, int launch_block, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_nn(locations, distances, numRecords);
    if (rc) return rc;
    return run_gptb_once(new OriNNKernel(0, (LatLong *)const_cast<float *>(locations), distances, numRecords, lat, lng),
                         block_start, block_end, launch_grid, launch_block, stream);
}

int tacker_hot3d_coefficients(int nx, int ny, int nz, float out[8])
{
    if (nx <= 0 || ny <= 0 || nz <= 0 || !out) return fail(TK_ERROR_INVALID_VALUE, "hot3d_coefficients: bad arguments");
    OriHOT3DParamsStruct q{};
    hot3dCoefficients(nx, ny, nz, &q);
    const float v[8] = {q.sdc, q.ce, q.cw, q.cn, q.cs, q.ct, q.cb, q.cc};
    for (int i = 0; i < 8; ++i) out[i] = v[i];
    return TK_SUCCESS;
}

int tacker_ori_hot3d(const float *p, const float *tIn, float *tOut, int nx, int ny, int nz, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_hot3d(p, tIn, tOut, nx, ny, nz);
    if (rc) return rc;
    return run_once(new OriHOT3DKernel(0, const_cast<float *>(p), const_cast<float *>(tIn), tOut, nx, ny, nz), stream);
}

int tacker_gptb_hot3d(const float *p, const float *tIn, float *tOut, int nx, int ny, int nz, int block_start,
                      int block_end, int launch_grid, int launch_block, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_hot3d(p, tIn, tOut, nx, ny, nz);
    if (rc) return rc;
    return run_gptb_once(new OriHOT3DKernel(0, const_cast<float *>(p), const_cast<float *>(tIn), tOut, nx, ny, nz),
                         block_start, block_end, launch_grid, launch_block, stream);
}

namespace {
int check_lava(int boxes1d, const float *rv, const float *qv, float *fv)
{
    if (!rv || !qv || !fv || rv == fv) return fail(TK_ERROR_INVALID_VALUE, "lava: bad arguments");
    if (boxes1d < 1 || boxes1d > 128) return fail(TK_ERROR_UNSUPPORTED, "lava: 1 .. 128 boxes along an edge");
    if ((((size_t)rv | (size_t)fv) & 15) != 0) return fail(TK_ERROR_INVALID_VALUE, "lava: rv and fv must be 16-byte aligned");
    return TK_SUCCESS;
}
Kernel *new_lava(float alpha, int boxes1d, const float *rv, const float *qv, float *fv, int *rc)
{
    Kernel *ori = nullptr;   // the box list is allocated and copied: not outside guarded()
    *rc = guarded([&]() -> int {
        ori = new OriLAVAKernel(0, alpha, boxes1d, (FOUR_VECTOR *)const_cast<float *>(rv), const_cast<float *>(qv),
                                (FOUR_VECTOR *)fv);
        return TK_SUCCESS;
    });
    return ori;
}
}  // namespace

int tacker_lava_blocks(int boxes1d) { return boxes1d < 1 || boxes1d > 128 ? 0 : boxes1d * boxes1d * boxes1d * LAVA_PARTS; }

int tacker_lava_boxes(int boxes1d, void *out, size_t out_bytes)
{
    if (boxes1d < 1 || boxes1d > 128 || !out) return fail(TK_ERROR_INVALID_VALUE, "lava_boxes: bad arguments");
    const std::vector<box_str> boxes = lavaBoxes(boxes1d);
    if (out_bytes < boxes.size() * sizeof(box_str)) return fail(TK_ERROR_INVALID_VALUE, "lava_boxes: buffer too small");
    memcpy(out, boxes.data(), boxes.size() * sizeof(box_str));
    return TK_SUCCESS;
}

int tacker_ori_lava(float alpha, int boxes1d, const float *rv, const float *qv, float *fv, tkStream_t stream)
{
    REQUIRE_INIT();
    int rc = check_lava(boxes1d, rv, qv, fv);
    if (rc) return rc;
    Kernel *ori = new_lava(alpha, boxes1d, rv, qv, fv, &rc);
    if (rc) return rc;
    return run_once(ori, stream);
}

int tacker_gptb_lava(float alpha, int boxes1d, const float *rv, const float *qv, float *fv, int block_start,
                     int block_end, int launch_grid, int launch_block, tkStream_t stream)
{
    REQUIRE_INIT();
    int rc = check_lava(boxes1d, rv, qv, fv);
    if (rc) return rc;
    Kernel *ori = new_lava(alpha, boxes1d, rv, qv, fv, &rc);
    if (rc) return rc;
    return run_gptb_once(ori, block_start, block_end, launch_grid, launch_block, stream);
}

int tacker_path_blocks(int cols, int iteration) { return pathBlocks(cols, iteration); }

int tacker_ori_path(int iteration, const int *wall, const int *src, int *results, int cols, int rows, int startStep,
                    tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_path(iteration, wall, src, results, cols, rows, startStep);
    if (rc) return rc;
    return run_once(new OriPATHKernel(0, iteration, const_cast<int *>(wall), const_cast<int *>(src), results, cols, rows,
                                      startStep),
                    stream);
}

int tacker_gptb_path(int iteration, const int *wall, const int *src, int *results, int cols, int rows, int startStep,
                     int block_start, int block_end, int launch_grid, int launch_block, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_path(iteration, wall, src, results, cols, rows, startStep);
    if (rc) return rc;
    return run_gptb_once(new OriPATHKernel(0, iteration, const_cast<int *>(wall), const_cast<int *>(src), results, cols,
                                           rows, startStep),
                         block_start, block_end, launch_grid, launch_block, stream);
}

namespace {
int check_cutcp(int binDim_x, int binDim_y, const float *binZeroAddr, float h, const float *regionZeroAddr, int rx,
                int ry, int rz)
{
    if (!binZeroAddr || !regionZeroAddr || binDim_x <= 0 || binDim_y <= 0 || !(h > 0) || rx <= 0 || ry <= 0 || rz <= 0)
        return fail(TK_ERROR_INVALID_VALUE, "cutcp: bad arguments");
    if ((long long)rx * ry * rz * REGION_SIZE >= (1ll << 31))
        return fail(TK_ERROR_UNSUPPORTED, "cutcp: a lattice of 2^31 points or more");
    return TK_SUCCESS;
}
}  // namespace

int tacker_cutcp_prepare_input(const float *atoms, int natoms, const float lo[3], int nx, int ny, int nz, float h,
                               float cutoff, int binDim[3], int *padding, float *bins, int *nbr, int *nbr_len,
                               int counts[2])
{
    if ((natoms > 0 && !atoms) || natoms < 0 || !lo || nx <= 0 || ny <= 0 || nz <= 0 || !(h > 0) || !(cutoff > 0) || !binDim ||
        !padding || !nbr_len)
        return fail(TK_ERROR_INVALID_VALUE, "cutcp_prepare_input: bad arguments");
    return guarded([&]() -> int {
        CutcpBins out;
        const char *why = nullptr;
        if (!cutcpPrepareInput(atoms, natoms, lo, nx, ny, nz, h, cutoff, &out, &why)) return fail(TK_ERROR_UNSUPPORTED, why);
        for (int d = 0; d < 3; ++d) binDim[d] = out.binDim[d];
        *padding = out.padding;
        *nbr_len = (int)out.nbrlist.size() / 3;
        if (bins) std::copy(out.bins.begin(), out.bins.end(), bins);
        if (nbr) std::copy(out.nbrlist.begin(), out.nbrlist.end(), nbr);
        if (counts) counts[0] = out.extra, counts[1] = out.excluded;
        return TK_SUCCESS;
    });
}

int tacker_cutcp_set_neighbours(const int *ijk, int len)
{
    REQUIRE_INIT();
    if (len < 0 || len > NBRLIST_MAXLEN || (len > 0 && !ijk))
        return fail(TK_ERROR_INVALID_VALUE, "cutcp: neighbour list length out of range");
    const int rc = cutcpSetNeighbours(ijk, len);
    return rc ? fail(rc, "cutcp: loading the neighbour list failed") : rc;
}

int tacker_cutcp_blocks(int rx, int ry, int rz)
{
    static_assert(TACKER_CUTCP_NBR_CHUNK == CUTCP_NBR_CHUNK, "public and device chunk sizes must agree");
    if (rx <= 0 || ry <= 0 || rz <= 0) return 0;
    return rx * ry * rz * cutcpNeighbourParts();
}

int tacker_ori_cutcp(int binDim_x, int binDim_y, const float *binZeroAddr, float h, float cutoff2, float inv_cutoff2,
                     float *regionZeroAddr, int rx, int ry, int rz, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_cutcp(binDim_x, binDim_y, binZeroAddr, h, regionZeroAddr, rx, ry, rz);
    if (rc) return rc;
    return run_once(new OriCUTCPKernel(0, binDim_x, binDim_y, const_cast<float *>(binZeroAddr), h, cutoff2, inv_cutoff2,
                                       regionZeroAddr, rx, ry, rz), stream);
}

int tacker_gptb_cutcp(int binDim_x, int binDim_y, const float *binZeroAddr, float h, float cutoff2, float inv_cutoff2,
                      float *regionZeroAddr, int rx, int ry, int rz, int block_start, int block_end, int launch_grid,
                      int launch_block, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_cutcp(binDim_x, binDim_y, binZeroAddr, h, regionZeroAddr, rx, ry, rz);
    if (rc) return rc;
    return run_gptb_once(new OriCUTCPKernel(0, binDim_x, binDim_y, const_cast<float *>(binZeroAddr), h, cutoff2,
                                            inv_cutoff2, regionZeroAddr, rx, ry, rz),
                         block_start, block_end, launch_grid, launch_block, stream);
}

int tacker_cp_set_atoms(const float *atoms_host, int count, float zplane)
{
    REQUIRE_INIT();
    if (!atoms_host || count < 0 || count > MAXATOMS) return fail(TK_ERROR_INVALID_VALUE, "cp: atom count out of range");
    const int rc = cpCopyAtomsToConstBuf(atoms_host, count, zplane);
    return rc ? fail(rc < 0 ? TK_ERROR_INVALID_VALUE : rc, "cp: loading the atom table failed") : rc;
}

int tacker_cp_initatoms(float *atoms_host, int count, unsigned volx, unsigned voly, unsigned volz, float gridspacing)
{
    if (!atoms_host || count < 0) return fail(TK_ERROR_INVALID_VALUE, "cp_initatoms: bad arguments");
    cpInitAtoms(atoms_host, count, volx, voly, volz, gridspacing);
    return TK_SUCCESS;
}

int tacker_cp_blocks(int volx, int voly)
{
    static_assert(TACKER_CP_X_PARTS == CP_X_PARTS, "public and device part counts must agree");
    if (volx < 0 || voly < 0) return 0;
    return (volx / (BLOCKSIZEX * UNROLLX)) * (voly / BLOCKSIZEY) * CP_X_PARTS;
}

int tacker_cp_inv_sqrt_selftest(unsigned lo_bits, unsigned hi_bits, unsigned long long *mismatches)
{
    REQUIRE_INIT();
    if (!mismatches || hi_bits < lo_bits) return fail(TK_ERROR_INVALID_VALUE, "cp_inv_sqrt_selftest: bad arguments");
    auto it = fmap.find("cp_inv_sqrt_selftest");
    if (it == fmap.end()) return fail(TK_ERROR_NOT_FOUND, "no kernel {cp_inv_sqrt_selftest}");
    return guarded([&]() -> int {
        unsigned long long *count = nullptr;
        TK_SAFE_CALL(tkMalloc((void **)&count, sizeof(*count)));
        TK_SAFE_CALL(tkMemset(count, 0, sizeof(*count)));
        void *args[] = {&lo_bits, &hi_bits, &count};
        const int rc = tkLaunchKernel(it->second, dim3(cuCount() * 8, 1, 1).raw(), dim3(256, 1, 1).raw(), args, 0,
                                      nullptr);
        if (rc == TK_SUCCESS) {
            TK_SAFE_CALL(tkDeviceSynchronize());
            TK_SAFE_CALL(tkMemcpy(mismatches, count, sizeof(*count), TK_MEMCPY_D2H));
        }
        tkErrCheck(tkFree(count));
        return rc;
    });
}

int tacker_ori_cp(int numatoms, float gridspacing, float *energygrid, int volx, int voly, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_cp(numatoms, energygrid, volx, voly);
    if (rc) return rc;
    return run_once(new OriCPKernel(0, numatoms, gridspacing, energygrid, volx, voly), stream);
}

int tacker_gptb_cp(int numatoms, float gridspacing, float *energygrid, int volx, int voly, int block_start,
                   int block_end, int launch_grid, int launch_block, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_cp(numatoms, energygrid, volx, voly);
    if (rc) return rc;
    return run_gptb_once(new OriCPKernel(0, numatoms, gridspacing, energygrid, volx, voly), block_start, block_end,
                         launch_grid, launch_block, stream);
}

int tacker_mix_tzgemm_stencil(float c0, float c1, const float *A0, float *Anext, int nx, int ny, int nz,
                              int be_start, int be_end, const void *A, const void *B, float *C, int M, int N,
                              int K, int tile_start, int tile_end, const char *variant, int launch_grid,
                              int launch_block, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_stencil(A0, Anext, nx, ny, nz);
    if (rc) return rc;
    return run_mix_once(new OriSTENCILKernel(0, c0, c1, A0, Anext, nx, ny, nz), be_start, be_end, A, B, C, M, N, K,
                        tile_start, tile_end, variant, launch_grid, launch_block, stream);
}

int tacker_mix_tzgemm_lbm(const float *src, float *dst, int sx, int sy, int sz, int be_start, int be_end,
                          const void *A, const void *B, float *C, int M, int N, int K, int tile_start,
                          int tile_end, const char *variant, int launch_grid, int launch_block, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_lbm(src, dst, sx, sy, sz);
    if (rc) return rc;
    return run_mix_once(new OriLBMKernel(0, src, dst, sx, sy, sz), be_start, be_end, A, B, C, M, N, K, tile_start,
                        tile_end, variant, launch_grid, launch_block, stream);
}

int tacker_mix_tzgemm_mriq(int numK, const float *x, const float *y, const float *z, float *Qr, float *Qi,
                           int numX, int be_start, int be_end, const void *A, const void *B, float *C, int M,
                           int N, int K, int tile_start, int tile_end, const char *variant, int launch_grid,
                           int launch_block, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_mriq(numK, x, y, z, Qr, Qi, numX);
    if (rc) return rc;
    return run_mix_once(new OriMRIQKernel(0, numK, x, y, z, Qr, Qi, numX), be_start, be_end, A, B, C, M, N, K,
                        tile_start, tile_end, variant, launch_grid, launch_block, stream);
}

int tacker_mix_tzgemm_mrif(int numK, const float *x, const float *y, const float *z, float *outR, float *outI,
                           int numX, int be_start, int be_end, const void *A, const void *B, float *C, int M,
                           int N, int K, int tile_start, int tile_end, const char *variant, int launch_grid,
                           int launch_block, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_mrif(numK, x, y, z, outR, outI, numX);
    if (rc) return rc;
    return run_mix_once(new OriMRIFKernel(0, numK, x, y, z, outR, outI, numX), be_start, be_end, A, B, C, M, N, K,
                        tile_start, tile_end, variant, launch_grid, launch_block, stream);
}

int tacker_mix_tzgemm_sgemm(const float *sA, const float *sB, float *sC, int sM, int sN, int sK, int be_start,
                            int be_end, const void *A, const void *B, float *C, int M, int N, int K, int tile_start,
                            int tile_end, const char *variant, int launch_grid, int launch_block, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_sgemm(sA, sB, sC, sM, sN, sK);
    if (rc) return rc;
    Kernel *ori = nullptr;
    const int made = guarded([&]() -> int {
        ori = new OriSGEMMKernel(0, sA, sB, sC, sM, sN, sK);
        return TK_SUCCESS;
    });
    if (made) return made;
    return run_mix_once(ori, be_start, be_end, A, B, C, M, N, K, tile_start, tile_end, variant, launch_grid,
                        launch_block, stream);
}

int tacker_mix_tzgemm_cutcp(int binDim_x, int binDim_y, const float *binZeroAddr, float h, float cutoff2,
                            float inv_cutoff2, float *regionZeroAddr, int rx, int ry, int rz, int be_start, int be_end,
                            const void *A, const void *B, float *C, int M, int N, int K, int tile_start, int tile_end,
                            const char *variant, int launch_grid, int launch_block, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_cutcp(binDim_x, binDim_y, binZeroAddr, h, regionZeroAddr, rx, ry, rz);
    if (rc) return rc;
    return run_mix_once(new OriCUTCPKernel(0, binDim_x, binDim_y, const_cast<float *>(binZeroAddr), h, cutoff2,
                                           inv_cutoff2, regionZeroAddr, rx, ry, rz),
                        be_start, be_end, A, B, C, M, N, K, tile_start, tile_end, variant, launch_grid, launch_block, stream);
}

int tacker_mix_tzgemm_fft(float *data, int batches, int be_start, int be_end, const void *A, const void *B, float *C,
                          int M, int N, int K, int tile_start, int tile_end, const char *variant, int launch_grid,
                          int launch_block, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_fft(data, batches);
    if (rc) return rc;
    return run_mix_once(new OriFFTKernel(0, data, batches), be_start, be_end, A, B, C, M, N, K, tile_start, tile_end,
                        variant, launch_grid, launch_block, stream);
}

int tacker_mix_tzgemm_nn(const float *locations, float *distances, int numRecords, float lat, float lng, int be_start,
                         int be_end, const void *A, const void *B, float *C, int M, int N, int K, int tile_start,
                         int tile_end, const char *variant, int launch_grid, int launch_block, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_nn(locations, distances, numRecords);
    if (rc) return rc;
    return run_mix_once(new OriNNKernel(0, (LatLong *)const_cast<float *>(locations), distances, numRecords, lat, lng),
                        be_start, be_end, A, B, C, M, N, K, tile_start, tile_end, variant, launch_grid, launch_block, stream);
}

int tacker_mix_tzgemm_hot3d(const float *p, const float *tIn, float *tOut, int nx, int ny, int nz, int be_start,
                            int be_end, const void *A, const void *B, float *C, int M, int N, int K, int tile_start,
                            int tile_end, const char *variant, int launch_grid, int launch_block, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_hot3d(p, tIn, tOut, nx, ny, nz);
    if (rc) return rc;
    return run_mix_once(new OriHOT3DKernel(0, const_cast<float *>(p), const_cast<float *>(tIn), tOut, nx, ny, nz),
                        be_start, be_end, A, B, C, M, N, K, tile_start, tile_end, variant, launch_grid, launch_block, stream);
}

int tacker_mix_tzgemm_lava(float alpha, int boxes1d, const float *rv, const float *qv, float *fv, int be_start,
                           int be_end, const void *A, const void *B, float *C, int M, int N, int K, int tile_start,
                           int tile_end, const char *variant, int launch_grid, int launch_block, tkStream_t stream)
{
    REQUIRE_INIT();
    int rc = check_lava(boxes1d, rv, qv, fv);
    if (rc) return rc;
    Kernel *ori = new_lava(alpha, boxes1d, rv, qv, fv, &rc);
    if (rc) return rc;
    return run_mix_once(ori, be_start, be_end, A, B, C, M, N, K, tile_start, tile_end, variant, launch_grid,
                        launch_block, stream);
}

int tacker_mix_tzgemm_path(int iteration, const int *wall, const int *src, int *results, int cols, int rows,
                           int startStep, int be_start, int be_end, const void *A, const void *B, float *C, int M,
                           int N, int K, int tile_start, int tile_end, const char *variant, int launch_grid,
                           int launch_block, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_path(iteration, wall, src, results, cols, rows, startStep);
    if (rc) return rc;
    return run_mix_once(new OriPATHKernel(0, iteration, const_cast<int *>(wall), const_cast<int *>(src), results, cols,
                                          rows, startStep),
                        be_start, be_end, A, B, C, M, N, K, tile_start, tile_end, variant, launch_grid, launch_block, stream);
}

int tacker_mix_tzgemm_cp(int numatoms, float gridspacing, float *energygrid, int volx, int voly, int be_start,
                         int be_end, const void *A, const void *B, float *C, int M, int N, int K, int tile_start,
                         int tile_end, const char *variant, int launch_grid, int launch_block, tkStream_t stream)
{
    REQUIRE_INIT();
    const int rc = check_cp(numatoms, energygrid, volx, voly);
    if (rc) return rc;
    return run_mix_once(new OriCPKernel(0, numatoms, gridspacing, energygrid, volx, voly), be_start, be_end, A, B, C,
                        M, N, K, tile_start, tile_end, variant, launch_grid, launch_block, stream);
}

int tacker_im2col(const float *data_im, int channels, int height, int width, int kernel_h, int kernel_w,
                  int pad_h, int pad_w, int stride_h, int stride_w, int dilation_h, int dilation_w,
                  float *data_col, tkStream_t stream)
{
    REQUIRE_INIT();
    if (!data_im || !data_col || channels < 1 || height < 1 || width < 1 || kernel_h < 1 || kernel_w < 1 ||
        stride_h < 1 || stride_w < 1 || dilation_h < 1 || dilation_w < 1 || pad_h < 0 || pad_w < 0)
        return fail(TK_ERROR_INVALID_VALUE, "im2col: bad arguments");
    int height_col = (height + 2 * pad_h - (dilation_h * (kernel_h - 1) + 1)) / stride_h + 1;
    int width_col = (width + 2 * pad_w - (dilation_w * (kernel_w - 1) + 1)) / stride_w + 1;
    if (height_col < 1 || width_col < 1) return fail(TK_ERROR_INVALID_VALUE, "im2col: empty output");
    int n = channels * height_col * width_col;
    int im_size = channels * height * width;
    int col_size = channels * kernel_h * kernel_w * height_col * width_col;
    void *args[] = {&n, &data_im, &height, &width, &kernel_h, &kernel_w, &pad_h, &pad_w, &stride_h, &stride_w,
                    &dilation_h, &dilation_w, &height_col, &width_col, &data_col, &im_size, &col_size};
    // grid-stride launch: 2 workgroups of 256 per CU, as the reference's SM_NUM*2
    const int rc = tkLaunchKernel(fmap["im2col"], dim3(cuCount() * 2).raw(), dim3(256).raw(), args, 0, stream);
    return rc ? fail(rc, tkGetErrorString(rc)) : rc;
}

int tacker_convert_fp32_to_fp16(void *out_f16, const float *in, int n, tkStream_t stream)
{
    REQUIRE_INIT();
    if (!out_f16 || !in || n < 0) return fail(TK_ERROR_INVALID_VALUE, "convert: bad arguments");
    if (n == 0) return TK_SUCCESS;
    void *args[] = {&out_f16, &in, &n};
    const int rc = tkLaunchKernel(fmap["convert_fp32_to_fp16"], dim3((n + 255) / 256).raw(), dim3(256).raw(), args, 0, stream);
    return rc ? fail(rc, tkGetErrorString(rc)) : rc;
}

int tacker_mnk_from_conv_args(const int a[14], int mnk[3])
{
    const int height_col = (a[2] + 2 * a[8] - (a[12] * (a[6] - 1) + 1)) / a[10] + 1;
    const int width_col = (a[3] + 2 * a[9] - (a[13] * (a[7] - 1) + 1)) / a[11] + 1;
    mnk[0] = a[0] * height_col * width_col;
    mnk[1] = a[4];
    mnk[2] = a[6] * a[7] * a[1];
    return TK_SUCCESS;
}

int tacker_get_kernel_info(const char *kernel, const char *key) { return get_kernel_info(kernel, key); }
float tacker_fget_kernel_info(const char *kernel, const char *key) { return fget_kernel_info(kernel, key); }

// ---- object API -------------------------------------------------------------

tacker_kernel_t tacker_create_kernel(const char *name)
{
    if (!tacker_runtime_ready() || !name) {
        fail(TK_ERROR_INVALID_VALUE, "tacker_create_kernel: not initialised");
        return nullptr;
    }
    static const char *known[] = {"cp",   "cutcp", "fft", "hot3d", "lava",  "lbm",     "mrif",
                                  "mriq", "nn",    "path", "sgemm", "stencil", "tzgemm"};
    bool ok = false;
    for (auto k : known) ok |= (strcmp(k, name) == 0);
    if (!ok) {
        fail(TK_ERROR_NOT_FOUND, std::string("Creator: Kernel not found: ") + name);
        return nullptr;
    }
    tacker_kernel_t out = nullptr;
    guarded([&]() -> int {
        out = static_cast<Kernel *>(createKernel(name));
        return TK_SUCCESS;
    });
    return out;
}

#define CREATE(check_expr, new_expr)                          \
    do {                                                      \
        if (!tacker_runtime_ready()) {                        \
            fail(TK_ERROR_INVALID_VALUE, "not initialised");  \
            return nullptr;                                   \
        }                                                     \
        if (check_expr) return nullptr;                       \
        tacker_kernel_t out_ = nullptr;                       \
        guarded([&]() -> int {                                         \
            out_ = static_cast<Kernel *>(new_expr);           \
            return TK_SUCCESS;                                \
        });                                                   \
        return out_;                                          \
    } while (0)

tacker_kernel_t tacker_ori_stencil_create(float c0, float c1, const float *A0, float *Anext, int nx, int ny, int nz)
{
    CREATE(check_stencil(A0, Anext, nx, ny, nz), new OriSTENCILKernel(0, c0, c1, A0, Anext, nx, ny, nz));
}
tacker_kernel_t tacker_ori_lbm_create(const float *src, float *dst, int sx, int sy, int sz)
{
    CREATE(check_lbm(src, dst, sx, sy, sz), new OriLBMKernel(0, src, dst, sx, sy, sz));
}
tacker_kernel_t tacker_ori_mriq_create(int numK, const float *x, const float *y, const float *z, float *Qr, float *Qi, int numX)
{
    CREATE(check_mriq(numK, x, y, z, Qr, Qi, numX), new OriMRIQKernel(0, numK, x, y, z, Qr, Qi, numX));
}
tacker_kernel_t tacker_ori_cutcp_create(int binDim_x, int binDim_y, const float *binZeroAddr, float h, float cutoff2,
                                        float inv_cutoff2, float *regionZeroAddr, int rx, int ry, int rz)
{
    CREATE(check_cutcp(binDim_x, binDim_y, binZeroAddr, h, regionZeroAddr, rx, ry, rz),
           new OriCUTCPKernel(0, binDim_x, binDim_y, const_cast<float *>(binZeroAddr), h, cutoff2, inv_cutoff2,
                              regionZeroAddr, rx, ry, rz));
}

tacker_kernel_t tacker_ori_fft_create(float *data, int batches)
{
    CREATE(check_fft(data, batches), new OriFFTKernel(0, data, batches));
}

tacker_kernel_t tacker_ori_nn_create(const float *locations, float *distances, int numRecords, float lat, float lng)
{
    CREATE(check_nn(locations, distances, numRecords),
           new OriNNKernel(0, (LatLong *)const_cast<float *>(locations), distances, numRecords, lat, lng));
}

tacker_kernel_t tacker_ori_hot3d_create(const float *p, const float *tIn, float *tOut, int nx, int ny, int nz)
{
    CREATE(check_hot3d(p, tIn, tOut, nx, ny, nz),
           new OriHOT3DKernel(0, const_cast<float *>(p), const_cast<float *>(tIn), tOut, nx, ny, nz));
}

tacker_kernel_t tacker_ori_lava_create(float alpha, int boxes1d, const float *rv, const float *qv, float *fv)
{
    CREATE(check_lava(boxes1d, rv, qv, fv),
           new OriLAVAKernel(0, alpha, boxes1d, (FOUR_VECTOR *)const_cast<float *>(rv), const_cast<float *>(qv),
                             (FOUR_VECTOR *)fv));
}

tacker_kernel_t tacker_ori_path_create(int iteration, const int *wall, const int *src, int *results, int cols, int rows,
                                       int startStep)
{
    CREATE(check_path(iteration, wall, src, results, cols, rows, startStep),
           new OriPATHKernel(0, iteration, const_cast<int *>(wall), const_cast<int *>(src), results, cols, rows, startStep));
}

tacker_kernel_t tacker_ori_sgemm_create(const float *A, const float *B, float *C, int M, int N, int K)
{
    CREATE(check_sgemm(A, B, C, M, N, K), new OriSGEMMKernel(0, A, B, C, M, N, K));
}

tacker_kernel_t tacker_ori_mrif_create(int numK, const float *x, const float *y, const float *z, float *outR, float *outI, int numX)
{
    CREATE(check_mrif(numK, x, y, z, outR, outI, numX), new OriMRIFKernel(0, numK, x, y, z, outR, outI, numX));
}
tacker_kernel_t tacker_ori_cp_create(int numatoms, float gridspacing, float *energygrid, int volx, int voly)
{
    CREATE(check_cp(numatoms, energygrid, volx, voly), new OriCPKernel(0, numatoms, gridspacing, energygrid, volx, voly));
}
tacker_kernel_t tacker_ori_tzgemm_create(const void *A, const void *B, float *C, int m, int n, int k)
{
    if (m < 1 || n < 1 || k < 1) {
        fail(TK_ERROR_INVALID_VALUE, "tzgemm: bad dimensions");
        return nullptr;
    }
    if (!A) CREATE(0, new OriTZGEMMKernel(0, m, n, k));
    CREATE((!B || !C) ? fail(TK_ERROR_INVALID_VALUE, "tzgemm: null operand") : 0, new OriTZGEMMKernel(0, m, n, k, A, B, C));
}

tacker_kernel_t tacker_gptb_create(tacker_kernel_t ori_handle, int launch_grid, int launch_block, int start, int end)
{
    Kernel *ori = static_cast<Kernel *>(ori_handle);
    if (!ori || dynamic_cast<GPTBKernel *>(ori) || dynamic_cast<MixKernel *>(ori)) {
        fail(TK_ERROR_INVALID_VALUE, "tacker_gptb_create: handle is not an ori kernel");
        return nullptr;
    }
    const int block = launch_block > 0 ? launch_block : (ori->kernelName == "tzgemm" ? TZ_THREADS : default_block(ori->kernelName));
    CREATE(check_range(ori, start, end) || check_block(ori->kernelName, block), make_gptb(ori, launch_grid, block, start, end));
}

int tacker_gptb_set_range(tacker_kernel_t h, int start, int end)
{
    GPTBKernel *g = dynamic_cast<GPTBKernel *>(static_cast<Kernel *>(h));
    if (!g) return fail(TK_ERROR_INVALID_VALUE, "not a GPTB kernel");
    const int rc = check_range(g->kernel_, start, end);
    if (rc) return rc;
    g->gptbParams.ptb_start_block_pos = start;
    g->gptbParams.ptb_end_block_pos = end;
    return TK_SUCCESS;
}

tacker_kernel_t tacker_mix_create(tacker_kernel_t be_h, tacker_kernel_t tz_h, int be_start, int be_end,
                                  int tile_start, int tile_end, const char *variant, int launch_grid, int launch_block)
{
    GPTBKernel *be = dynamic_cast<GPTBKernel *>(static_cast<Kernel *>(be_h));
    GPTBKernel *tz = dynamic_cast<GPTBKernel *>(static_cast<Kernel *>(tz_h));
    if (!be || !tz || tz->kernelName != "tzgemm" || be->kernelName == "tzgemm") {
        fail(TK_ERROR_INVALID_VALUE, "tacker_mix_create: need a best-effort GPTB kernel and a tzgemm GPTB kernel");
        return nullptr;
    }
    const std::string v = variant ? variant : "";
    const std::string key = "tzgemm_" + be->kernelName + (v.empty() ? "" : "@" + v);
    if (!has_key(key) || get_kernel_info(key, "blocksize") == JSON_NOT_FOUND) {
        fail(TK_ERROR_NOT_FOUND, "no fused kernel {" + key + "}");
        return nullptr;
    }
    if (launch_block > 0 && launch_block != get_kernel_info(key, "blocksize")) {
        fail(TK_ERROR_INVALID_VALUE, "{" + key + "} is built for another workgroup size");
        return nullptr;
    }
    CREATE(check_range(be->kernel_, be_start, be_end) || check_range(tz->kernel_, tile_start, tile_end),
           createTzgemmMix(be, tz, be_start, be_end, tile_start, tile_end, v, launch_grid, launch_block));
}

tacker_kernel_t tacker_be_pair_create(tacker_kernel_t first_h, tacker_kernel_t second_h, int start1, int end1,
                                      int start2, int end2, const char *variant, int launch_grid)
{
    GPTBKernel *a = dynamic_cast<GPTBKernel *>(static_cast<Kernel *>(first_h));
    GPTBKernel *b = dynamic_cast<GPTBKernel *>(static_cast<Kernel *>(second_h));
    if (!a || !b || a->kernelName == "tzgemm" || b->kernelName == "tzgemm" || !(a->kernelName < b->kernelName)) {
        fail(TK_ERROR_INVALID_VALUE,
             "tacker_be_pair_create: need two different best-effort GPTB kernels, first < second alphabetically");
        return nullptr;
    }
    const std::string v = variant ? variant : "";
    const std::string key = a->kernelName + "_" + b->kernelName + (v.empty() ? "" : "@" + v);
    if (!has_key(key) || get_kernel_info(key, "blocksize") == JSON_NOT_FOUND) {
        fail(TK_ERROR_NOT_FOUND, "no fused kernel {" + key + "}");
        return nullptr;
    }
    CREATE(check_range(a->kernel_, start1, end1) || check_range(b->kernel_, start2, end2),
           createBePairMix(a, b, start1, end1, start2, end2, v, launch_grid));
}

tacker_kernel_t tacker_create_mix_kernel(const char *name)
{
    const std::string n = name ? name : "";
    if (n.find('_') == std::string::npos || !has_key(n) || get_kernel_info(n, "blocksize") == JSON_NOT_FOUND ||
        n.rfind("tzgemm_", 0) == 0) {
        fail(TK_ERROR_NOT_FOUND, "createMixKernel: no best-effort pair {" + n + "}");
        return nullptr;
    }
    CREATE(TK_SUCCESS, createMixKernel(n));
}

int tacker_mix_set_range(tacker_kernel_t h, int be_start, int be_end, int tile_start, int tile_end)
{
    MixKernel *m = dynamic_cast<MixKernel *>(static_cast<Kernel *>(h));
    if (!m) return fail(TK_ERROR_INVALID_VALUE, "not a mix kernel");
    if (be_start < 0 || be_end < be_start || tile_start < 0 || tile_end < tile_start)
        return fail(TK_ERROR_INVALID_VALUE, "bad range");
    m->kernel1_start_block_pos = be_start;
    m->kernel1_end_block_pos = be_end;
    m->kernel2_start_block_pos = tile_start;
    m->kernel2_end_block_pos = tile_end;
    return TK_SUCCESS;
}

namespace {
int check_mix_call(GPTBKernel *be, int start, int end)
{
    if (!be) return fail(TK_ERROR_INVALID_VALUE, "the best-effort kernel must be a GPTB kernel object");
    if (dynamic_cast<OriTZGEMMKernel *>(be->kernel_))
        return fail(TK_ERROR_INVALID_VALUE, "the best-effort kernel cannot be the GEMM itself");
    if (start < 0 || end < start) return fail(TK_ERROR_INVALID_VALUE, "bad block range");
    return TK_SUCCESS;
}
}  // namespace

int tacker_mix_cublas_sgemm(const int mnk[3], tacker_kernel_t be_gptb, int cd_start_blk, int cd_end_blk,
                            tkStream_t stream)
{
    REQUIRE_INIT();
    GPTBKernel *be = dynamic_cast<GPTBKernel *>(static_cast<Kernel *>(be_gptb));
    const int rc = check_mix_call(be, cd_start_blk, cd_end_blk);
    if (rc) return rc;
    if (!mnk || mnk[0] <= 0 || mnk[1] <= 0 || mnk[2] <= 0) return fail(TK_ERROR_INVALID_VALUE, "bad GEMM dimensions");
    return guarded([&]() -> int {
        std::vector<int> args(mnk, mnk + 3);
        mixcublasSgemm(args, be, cd_start_blk, cd_end_blk, stream);
        return TK_SUCCESS;
    });
}

int tacker_mix_cudnn_convolution_forward(const int cudnn_args[14], tacker_kernel_t be_gptb, int cd_start_blk,
                                         int cd_end_blk, tkStream_t stream)
{
    REQUIRE_INIT();
    GPTBKernel *be = dynamic_cast<GPTBKernel *>(static_cast<Kernel *>(be_gptb));
    const int rc = check_mix_call(be, cd_start_blk, cd_end_blk);
    if (rc) return rc;
    if (!cudnn_args) return fail(TK_ERROR_INVALID_VALUE, "null convolution arguments");
    for (int i = 0; i < 14; ++i)
        if (cudnn_args[i] < (i == 8 || i == 9 ? 0 : 1)) return fail(TK_ERROR_INVALID_VALUE, "bad convolution arguments");
    std::vector<int> args(cudnn_args, cudnn_args + 14);
    const int *a = cudnn_args;   // the dilated filter must fit the padded image in both directions
    if (a[2] + 2 * a[8] < a[12] * (a[6] - 1) + 1 || a[3] + 2 * a[9] < a[13] * (a[7] - 1) + 1)
        return fail(TK_ERROR_INVALID_VALUE, "the filter does not fit the input");
    return guarded([&]() -> int {
        mixcudnnConvolutionForward(args, be, cd_start_blk, cd_end_blk, stream);
        return TK_SUCCESS;
    });
}

int tacker_register_module(const char *module_name, const char *code_object_path)
{
    REQUIRE_INIT();
    if (!module_name || !*module_name || !code_object_path) return fail(TK_ERROR_INVALID_VALUE, "null module name or path");
    if (!moduleCenter.registerModule(module_name, code_object_path))
        return fail(TK_ERROR_DEVICE, std::string("cannot load code object ") + code_object_path);
    return TK_SUCCESS;
}

int tacker_module_has_function(const char *module_name, const char *function_name)
{
    if (!module_name || !function_name) return 0;
    return moduleCenter.getFunction(module_name, function_name) != nullptr;
}

int tacker_kernel_use_module(tacker_kernel_t h, const char *module_name, const char *function_name)
{
    Kernel *k = static_cast<Kernel *>(h);
    if (!k || !module_name || !function_name) return fail(TK_ERROR_INVALID_VALUE, "null kernel, module or function name");
    if (!dynamic_cast<GPTBKernel *>(k) && !dynamic_cast<MixKernel *>(k))
        return fail(TK_ERROR_UNSUPPORTED, "only GPTB and fused kernel objects launch from a code object");
    if (!k->useModule(module_name, function_name))
        return fail(TK_ERROR_NOT_FOUND, std::string("no function ") + function_name + " in module " + module_name);
    return TK_SUCCESS;
}

int tacker_kernel_execute(tacker_kernel_t h, tkStream_t stream)
{
    Kernel *k = static_cast<Kernel *>(h);
    if (!k) return fail(TK_ERROR_INVALID_VALUE, "null kernel");
    if (dynamic_cast<OriTZGEMMKernel *>(k)) return fail(TK_ERROR_UNSUPPORTED, "the GEMM runs only in GPTB or fused form");
    return guarded([&]() -> int {
        k->execute(stream);
        return TK_SUCCESS;
    });
}

int tacker_kernel_swap_buffers(tacker_kernel_t h)
{
    Kernel *k = static_cast<Kernel *>(h);
    if (auto *g = dynamic_cast<GPTBKernel *>(k)) k = g->kernel_;
    if (auto *s = dynamic_cast<OriSTENCILKernel *>(k)) { s->swapGrids(); return TK_SUCCESS; }
    if (auto *l = dynamic_cast<OriLBMKernel *>(k)) { l->swapGrids(); return TK_SUCCESS; }
    return fail(TK_ERROR_INVALID_VALUE, "only stencil and lbm objects ping-pong");
}

int tacker_kernel_info(tacker_kernel_t h, int out[8])
{
    Kernel *k = static_cast<Kernel *>(h);
    if (!k) return fail(TK_ERROR_INVALID_VALUE, "null kernel");
    memset(out, 0, 8 * sizeof(int));
    out[0] = (int)k->launchGridDim.x;
    out[1] = (int)(k->launchBlockDim.x * k->launchBlockDim.y * k->launchBlockDim.z);
    out[4] = (int)k->kernelParams.size();
    out[5] = (int)k->smem;
    Kernel *ori = k;
    if (auto *g = dynamic_cast<GPTBKernel *>(k)) {
        out[2] = g->gptbParams.ptb_start_block_pos;
        out[3] = g->gptbParams.ptb_end_block_pos;
        ori = g->kernel_;
    }
    out[6] = (int)ori->launchGridDim.x;
    out[7] = (int)ori->launchGridDim.y;
    return TK_SUCCESS;
}

int tacker_kernel_param(tacker_kernel_t h, int index, void *out, int bytes)
{
    Kernel *k = static_cast<Kernel *>(h);
    if (!k || !out) return fail(TK_ERROR_INVALID_VALUE, "null kernel or output");
    if (index < 0 || (size_t)index >= k->kernelParams.size() || (bytes != 4 && bytes != 8))
        return fail(TK_ERROR_INVALID_VALUE, "parameter index out of range, or size not 4 or 8 bytes");
    memcpy(out, k->kernelParams[index], (size_t)bytes);
    return TK_SUCCESS;
}

int tacker_kernel_destroy(tacker_kernel_t h)
{
    delete static_cast<Kernel *>(h);
    return TK_SUCCESS;
}

int tacker_spin_fail_flag(int *flag)
{
    REQUIRE_INIT();
    if (!flag) return fail(TK_ERROR_INVALID_VALUE, "null output");
    unsigned v = 0, zero = 0;
    int rc = tkMemcpyFromSymbol(&v, "tk_spin_fail", sizeof(v), 0);
    if (!rc && v) rc = tkMemcpyToSymbol("tk_spin_fail", &zero, sizeof(zero), 0);
    *flag = (int)v;
    return rc ? fail(rc, tkGetErrorString(rc)) : rc;
}

uint16_t tacker_float_to_half_bits(float f) { return tk::float_to_half_bits(f); }

int tacker_rng_uniform(uint64_t seed, float lo, float hi, float *out, size_t n)
{
    if (!out) return fail(TK_ERROR_INVALID_VALUE, "null output");
    tk::Rng rng(seed);
    for (size_t i = 0; i < n; ++i) out[i] = rng.uniform(lo, hi);
    return TK_SUCCESS;
}


// ---- LC task and scheduler ----------------------------------------------------

tacker_task_t tacker_task_create(const char *model, int height, int width)
{
    if (!tacker_runtime_ready() || !model) {
        fail(TK_ERROR_INVALID_VALUE, "tacker_task_create: not initialised");
        return nullptr;
    }
    if (strcmp(model, "vgg16")) {
        fail(TK_ERROR_NOT_FOUND, std::string("createTask: model not found: ") + model);
        return nullptr;
    }
    VGG16Options opt;
    if (height > 0) opt.height = height;
    if (width > 0) opt.width = width;
    if (opt.height % 32 || opt.width % 32) {
        fail(TK_ERROR_UNSUPPORTED, "vgg16: input resolution must be a multiple of 32");
        return nullptr;
    }
    tacker_task_t out = nullptr;
    guarded([&]() -> int {
        out = static_cast<Task *>(new VGG16(1, opt));
        return TK_SUCCESS;
    });
    return out;
}

int tacker_task_destroy(tacker_task_t task)
{
    delete static_cast<Task *>(task);
    return TK_SUCCESS;
}

int tacker_task_execute(tacker_task_t h, tkStream_t stream)
{
    Task *t = static_cast<Task *>(h);
    if (!t) return fail(TK_ERROR_INVALID_VALUE, "null task");
    return guarded([&]() -> int {
        t->initExecution();
        for (auto *k : t->kernels) k->execute(stream);
        return TK_SUCCESS;
    });
}

int tacker_task_stage_input(tacker_task_t h)
{
    Task *t = static_cast<Task *>(h);
    if (!t) return fail(TK_ERROR_INVALID_VALUE, "null task");
    return guarded([&]() -> int {
        t->initExecution();
        return TK_SUCCESS;
    });
}

int tacker_task_capture(tacker_task_t h, tkStream_t stream, tkGraphExec_t *exec)
{
    Task *t = static_cast<Task *>(h);
    if (!t || !exec) return fail(TK_ERROR_INVALID_VALUE, "null task or result");
    if (!stream) return fail(TK_ERROR_INVALID_VALUE, "the null stream cannot record a graph");
    return guarded([&]() -> int {
        *exec = t->captureQuery(stream);
        return TK_SUCCESS;
    });
}

int tacker_task_kernel_count(tacker_task_t h)
{
    Task *t = static_cast<Task *>(h);
    return t ? (int)t->kernels.size() : -1;
}

int tacker_task_kernel_info(tacker_task_t h, int index, char *name, int name_cap, int *mixable, int args[14], int *nargs)
{
    Task *t = static_cast<Task *>(h);
    if (!t || index < 0 || index >= (int)t->kernels.size()) return fail(TK_ERROR_INVALID_VALUE, "bad kernel index");
    Kernel *k = t->kernels[index];
    if (name && name_cap > 0) snprintf(name, name_cap, "%s", k->kernelName.c_str());
    if (mixable) *mixable = (int)k->mixable;
    const std::vector<int> a = k->getArgs();
    if (nargs) *nargs = (int)a.size();
    if (args)
        for (size_t i = 0; i < a.size() && i < 14; ++i) args[i] = a[i];
    return TK_SUCCESS;
}

int tacker_task_activation(tacker_task_t h, int conv_index, float **ptr, int dims[4])
{
    VGG16 *v = dynamic_cast<VGG16 *>(static_cast<Task *>(h));
    if (!v || conv_index < 0 || conv_index >= 16) return fail(TK_ERROR_INVALID_VALUE, "bad activation index");
    const VGG16::Act a = v->activation(conv_index);
    *ptr = a.ptr;
    dims[0] = a.H; dims[1] = a.W; dims[2] = a.C; dims[3] = a.ld;
    return TK_SUCCESS;
}

int tacker_task_conv_params(tacker_task_t h, int conv_index, void **weights, float **bias, int dims[2])
{
    VGG16 *v = dynamic_cast<VGG16 *>(static_cast<Task *>(h));
    if (!v || conv_index < 0 || conv_index >= 16) return fail(TK_ERROR_INVALID_VALUE, "bad layer index");
    const VGG16::Act a = v->activation(conv_index);
    *weights = a.weights;
    *bias = a.bias;
    dims[0] = a.Np;
    dims[1] = a.Kp;
    return TK_SUCCESS;
}

int tacker_task_logits(tacker_task_t h, const float **ptr, long *stride, int *count)
{
    VGG16 *v = dynamic_cast<VGG16 *>(static_cast<Task *>(h));
    if (!v) return fail(TK_ERROR_INVALID_VALUE, "not a vgg16 task");
    *ptr = v->logits(stride);
    if (count) *count = v->opt.classes;
    return TK_SUCCESS;
}

int tacker_task_input(tacker_task_t h, float **host_ptr, int *bytes)
{
    Task *t = static_cast<Task *>(h);
    if (!t) return fail(TK_ERROR_INVALID_VALUE, "null task");
    *host_ptr = static_cast<float *>(t->InputHost[0]);
    *bytes = t->InputSize[0];
    return TK_SUCCESS;
}

tacker_task_manager_t tacker_task_manager_create(tacker_task_t lc_task, const char *be1, const char *be2)
{
    if (!lc_task || !be1) {
        fail(TK_ERROR_INVALID_VALUE, "tacker_task_manager_create: bad arguments");
        return nullptr;
    }
    // fused pairs of two best-effort kernels exist within a family only (src/Creator.cu:341-640)
    static const char *families[2][8] = {{"cp", "cutcp", "fft", "lbm", "mrif", "mriq", "sgemm", "stencil"},
                                         {"hot3d", "lava", "nn", "path", nullptr, nullptr, nullptr, nullptr}};
    int family1 = -1, family2 = (!be2 || !*be2) ? -2 : -1;
    for (int f = 0; f < 2; ++f)
        for (auto k : families[f]) {
            if (!k) continue;
            if (strcmp(k, be1) == 0) family1 = f;
            if (family2 == -1 && strcmp(k, be2) == 0) family2 = f;
        }
    if (family1 < 0 || family2 == -1) {
        fail(TK_ERROR_NOT_FOUND, "Creator: Kernel not found");
        return nullptr;
    }
    if (family2 >= 0 && family2 != family1) {
        fail(TK_ERROR_NOT_FOUND, std::string("Creator: no fused kernel of ") + be1 + " and " + be2);
        return nullptr;
    }
    return new TaskManager(static_cast<Task *>(lc_task), be1, be2 ? be2 : "");
}

int tacker_task_manager_destroy(tacker_task_manager_t tm)
{
    delete static_cast<TaskManager *>(tm);
    return TK_SUCCESS;
}

int tacker_task_manager_configure(tacker_task_manager_t h, float qos_budget_ms, float guard_ms, int warmup_queries,
                                  int profile_queries, int queries, int verbose)
{
    TaskManager *tm = static_cast<TaskManager *>(h);
    if (!tm) return fail(TK_ERROR_INVALID_VALUE, "null task manager");
    if (qos_budget_ms >= 0) tm->policy.qos_budget_ms = qos_budget_ms;
    if (guard_ms >= 0) tm->policy.guard_ms = guard_ms;
    if (warmup_queries >= 0) tm->warmup_queries = warmup_queries;
    if (profile_queries >= 0) tm->profile_queries = profile_queries;
    if (queries >= 0) tm->queries = queries;
    if (verbose >= 0) tm->verbose = verbose != 0;
    return TK_SUCCESS;
}

int tacker_task_manager_run(tacker_task_manager_t h, int mode, tkStream_t stream, int second_stage)
{
    TaskManager *tm = static_cast<TaskManager *>(h);
    if (!tm) return fail(TK_ERROR_INVALID_VALUE, "null task manager");
    if (mode != 0 && mode != 1) return fail(TK_ERROR_INVALID_VALUE, "mode must be 0 (Aker) or 1 (Tacker)");
    if (second_stage && tm->be_task2_name.empty()) return fail(TK_ERROR_INVALID_VALUE, "no second BE kernel");
    return guarded([&]() -> int {
        const ExecutionMode m = mode ? ExecutionMode::Tacker : ExecutionMode::Aker;
        if (second_stage) tm->executeAllTasks(m, stream);
        else tm->execute_with_one_cd_kernel(m, stream);
        return TK_SUCCESS;
    });
}

int tacker_task_manager_report(tacker_task_manager_t h, float out[13])
{
    TaskManager *tm = static_cast<TaskManager *>(h);
    if (!tm) return fail(TK_ERROR_INVALID_VALUE, "null task manager");
    const TaskManagerReport &r = tm->report;
    const float v[13] = {r.lc_solo_ms, r.be1_solo_ms, r.be2_solo_ms, (float)r.be_blocks_executed,
                         (float)r.mix_times, (float)r.mixable_times, r.time_earned_ms, r.qos_headroom_left_ms,
                         r.stage1_be_ms, r.stage2_be_ms, (float)tm->be_task_finish_num,
                         (float)r.query_latency_ms.size(), (float)r.solo_latency_ms.size()};
    memcpy(out, v, sizeof(v));
    return TK_SUCCESS;
}

int tacker_task_manager_set_fusion_strikes(tacker_task_manager_t h, int limit)
{
    TaskManager *tm = static_cast<TaskManager *>(h);
    if (!tm || limit < 0) return fail(TK_ERROR_INVALID_VALUE, "bad task manager or limit");
    tm->fusion_strikes_limit = limit;
    return TK_SUCCESS;
}

int tacker_task_manager_set_calibration(tacker_task_manager_t h, int on, float max_stretch)
{
    TaskManager *tm = static_cast<TaskManager *>(h);
    if (!tm || max_stretch < 0.0f) return fail(TK_ERROR_INVALID_VALUE, "bad task manager or stretch");
    tm->calibrate_blocks = on != 0;
    tm->calibrate_max_stretch = max_stretch;
    return TK_SUCCESS;
}

int tacker_task_manager_set_calibration_budget(tacker_task_manager_t h, float query_stretch, int passes)
{
    TaskManager *tm = static_cast<TaskManager *>(h);
    if (!tm || query_stretch < 0.0f || passes < 1) return fail(TK_ERROR_INVALID_VALUE, "bad task manager, stretch or passes");
    tm->calibrate_query_stretch = query_stretch;
    tm->calibrate_passes = passes;
    return TK_SUCCESS;
}

int tacker_task_manager_set_calibration_variants(tacker_task_manager_t h, const char *variants)
{
    TaskManager *tm = static_cast<TaskManager *>(h);
    if (!tm || !variants) return fail(TK_ERROR_INVALID_VALUE, "bad task manager or list");
    std::vector<std::string> forms;
    std::string item;
    for (const char *c = variants;; ++c) {
        if (*c == ',' || *c == 0) {
            forms.push_back(item == "default" ? std::string() : item);
            item.clear();
            if (*c == 0) break;
        } else {
            item.push_back(*c);
        }
    }
    tm->calibrate_variants = forms;
    return TK_SUCCESS;
}

int tacker_task_manager_calibrated_variant(tacker_task_manager_t h, int kernel, char *out, int cap)
{
    TaskManager *tm = static_cast<TaskManager *>(h);
    if (!tm || !out || cap < 1 || kernel < 0 || kernel >= (int)tm->calibrated_variant.size()) return -1;
    const std::string &v = tm->calibrated_variant[(size_t)kernel];
    snprintf(out, (size_t)cap, "%s", v.c_str());
    return (int)v.size();
}

int tacker_task_manager_set_end_to_end(tacker_task_manager_t h, int queries)
{
    TaskManager *tm = static_cast<TaskManager *>(h);
    if (!tm || queries < 0) return fail(TK_ERROR_INVALID_VALUE, "bad task manager handle or query count");
    tm->end_to_end_queries = queries;
    return TK_SUCCESS;
}

int tacker_task_manager_calibrated_blocks(tacker_task_manager_t h, int *out, int cap)
{
    TaskManager *tm = static_cast<TaskManager *>(h);
    if (!tm || !out) return -1;
    const int n = std::min((int)tm->calibrated_blocks.size(), cap);
    memcpy(out, tm->calibrated_blocks.data(), (size_t)n * sizeof(int));
    return n;
}

int tacker_task_manager_fusion_disabled(tacker_task_manager_t h)
{
    TaskManager *tm = static_cast<TaskManager *>(h);
    return tm ? tm->report.fusion_disabled : -1;
}

float tacker_task_manager_be_mix_ms(tacker_task_manager_t h)
{
    TaskManager *tm = static_cast<TaskManager *>(h);
    return tm ? tm->report.be_mix_ms : -1.0f;
}

int tacker_task_manager_latencies(tacker_task_manager_t h, int which, float *out, int cap)
{
    TaskManager *tm = static_cast<TaskManager *>(h);
    if (!tm || !out) return -1;
    const std::vector<float> *all[] = {&tm->report.query_latency_ms,      &tm->report.solo_latency_ms,
                                       &tm->report.e2e_colocated_ms,      &tm->report.e2e_solo_ms,
                                       &tm->report.e2e_colocated_wall_ms, &tm->report.e2e_solo_wall_ms,
                                       &tm->report.e2e_graph_ms,          &tm->report.e2e_graph_wall_ms};
    if (which < 0 || which > 7) return -1;
    const std::vector<float> &v = *all[which];
    const int n = std::min((int)v.size(), cap);
    memcpy(out, v.data(), (size_t)n * sizeof(float));
    return n;
}

float tacker_qos_block_ratio(const char *be_name, int K_GLOBAL) { return QosPolicy::blockRatio(be_name, K_GLOBAL); }
float tacker_qos_whole_kernel_gain(const char *be_name) { return QosPolicy::wholeKernelGain(be_name ? be_name : ""); }

int tacker_qos_colocated_blocks(int mode, const char *be_name, int tiles, int K_GLOBAL, int be_total_blocks)
{
    return QosPolicy::coLocatedBlocks(mode ? ExecutionMode::Tacker : ExecutionMode::Aker, be_name, tiles, K_GLOBAL,
                                      be_total_blocks);
}

int tacker_qos_must_run_solo(float budget_ms, float guard_ms, float qos_headroom, float lc_time_remaining)
{
    QosPolicy p;
    p.qos_budget_ms = budget_ms;
    p.guard_ms = guard_ms;
    return p.mustRunSolo(qos_headroom, lc_time_remaining) ? 1 : 0;
}

int tacker_qos_account(int mixable, float measured_ms, float solo_lc_ms, float be_ms, int cd_blocks,
                       int be_total_blocks, float out[3])
{
    const QosPolicy::Outcome o = QosPolicy::account((unsigned)mixable, measured_ms, solo_lc_ms, be_ms, cd_blocks,
                                                    be_total_blocks);
    out[0] = o.counted_as_mixed ? 1.0f : 0.0f;
    out[1] = o.charged_ms;
    out[2] = o.earned_ms;
    return TK_SUCCESS;
}

}  // extern "C"
