#include "Creator.h"

#include <unordered_map>

#include "Logger.h"
#include "json.h"

extern Logger logger;

static std::unordered_map<std::string, GPTBKernel *> kernelMap;
static std::unordered_map<std::string, MixKernel *> mixKernelMap;

int cuCount()
{
    static int cus = 0;
    if (!cus) TK_SAFE_CALL(tkGetCuCount(&cus));
    return cus;
}

// per-CU instances and block size of the plain GPTB launch of a kernel, from kinfo
static dim3 gptbGrid(const std::string &name)
{
    int per_cu = get_kernel_info(name, "solo_ptb_blks");
    if (per_cu == JSON_NOT_FOUND || per_cu < 1) per_cu = 1;
    return dim3(cuCount() * per_cu, 1, 1);
}
static dim3 gptbBlock(const std::string &name, int fallback)
{
    int bs = get_kernel_info(name, "blocksize");
    if (bs == JSON_NOT_FOUND || bs < 64) bs = fallback;
    return dim3(bs, 1, 1);
}
static int oriBlocks(const std::string &name, Kernel *ori)
{
    const int natural = (int)(ori->launchGridDim.x * ori->launchGridDim.y * ori->launchGridDim.z);
    const int v = get_kernel_info(name, "ori_blks");
    return v == JSON_NOT_FOUND ? natural : v;
}

GPTBKernel *createKernel(const std::string &name)
{
    auto hit = kernelMap.find(name);
    if (hit != kernelMap.end()) return hit->second;

    GPTBKernel *k = nullptr;
    if (name == "cp") {
        auto *ori = new OriCPKernel(10);
        k = new GPTBKernel(10, "cp", "gptb_cp", ori, gptbGrid(name), gptbBlock(name, 128), 0, oriBlocks(name, ori));
    } else if (name == "cutcp") {
        auto *ori = new OriCUTCPKernel(11);
        k = new GPTBKernel(11, "cutcp", "gptb_cutcp", ori, gptbGrid(name), gptbBlock(name, 128), 0, oriBlocks(name, ori));
    } else if (name == "nn") {
        // the reference gives all its Rodinia kernels the id 20 (src/Creator.cu:193-246)
        auto *ori = new OriNNKernel(20);
        k = new GPTBKernel(20, "nn", "gptb_nn", ori, gptbGrid(name), gptbBlock(name, 256), 0, oriBlocks(name, ori));
    } else if (name == "hot3d") {
        auto *ori = new OriHOT3DKernel(20);
        k = new GPTBKernel(20, "hot3d", "gptb_hot3d", ori, gptbGrid(name), gptbBlock(name, 256), 0, oriBlocks(name, ori));
    } else if (name == "lava") {
        auto *ori = new OriLAVAKernel(20);
        k = new GPTBKernel(20, "lava", "gptb_lava", ori, gptbGrid(name), gptbBlock(name, 256), 0, oriBlocks(name, ori));
    } else if (name == "path") {
        auto *ori = new OriPATHKernel(20);
        k = new GPTBKernel(20, "path", "gptb_path", ori, gptbGrid(name), gptbBlock(name, 256), 0, oriBlocks(name, ori));
    } else if (name == "fft") {
        auto *ori = new OriFFTKernel(12);
        k = new GPTBKernel(12, "fft", "gptb_fft", ori, gptbGrid(name), gptbBlock(name, 256), 0, oriBlocks(name, ori));
    } else if (name == "lbm") {
        auto *ori = new OriLBMKernel(16);
        k = new GPTBKernel(16, "lbm", "gptb_lbm", ori, gptbGrid(name), gptbBlock(name, 256), 0, oriBlocks(name, ori));
    } else if (name == "mriq") {
        auto *ori = new OriMRIQKernel(18);
        k = new GPTBKernel(18, "mriq", "gptb_mriq", ori, gptbGrid(name), gptbBlock(name, 256), 0, oriBlocks(name, ori));
    } else if (name == "mrif") {
        auto *ori = new OriMRIFKernel(17);
        k = new GPTBKernel(17, "mrif", "gptb_mrif", ori, gptbGrid(name), gptbBlock(name, 256), 0, oriBlocks(name, ori));
    } else if (name == "sgemm") {
        auto *ori = new OriSGEMMKernel(21);
        k = new GPTBKernel(21, "sgemm", "gptb_sgemm", ori, gptbGrid(name), gptbBlock(name, 128), 0, oriBlocks(name, ori));
    } else if (name == "stencil") {
        auto *ori = new OriSTENCILKernel(19);
        k = new GPTBKernel(19, "stencil", "gptb_stencil", ori, gptbGrid(name), gptbBlock(name, 256), 0, oriBlocks(name, ori));
    } else if (name == "tzgemm") {
        // the stand-alone GEMM job of the reference: 12800 x 512 x 4096
        auto *ori = new OriTZGEMMKernel(20, 12800, 512, 4096);
        k = new GPTBKernel(20, "tzgemm", "gptb_tzgemm", ori, gptbGrid(name), dim3(TZ_THREADS, 1, 1), 0,
                           getTZGEMMGridDim(12800, 512, 4096)[3]);
    } else {
        logger.ERROR("Creator: Kernel not found: " + name);
    }
    kernelMap[name] = k;
    return k;
}

MixKernel *createTzgemmMix(GPTBKernel *be, GPTBKernel *tz, int be_start, int be_end, int tile_start,
                           int tile_end, const std::string &variant, int launch_grid, int launch_block)
{
    const std::string base = "tzgemm_" + be->kernelName;
    std::string key = variant.empty() ? base : base + "@" + variant;
    if (variant.empty() && tz->kernel_) {
        // a GEMM large enough for 256 x 128 tiles takes the form kinfo names for such shapes, if the pair has one
        const std::vector<int> mnk = tz->kernel_->getArgs();
        if (mnk.size() == 3) {
            const std::vector<int> d = getTZGEMMGridDim(mnk[0], mnk[1], mnk[2]);
            const std::string large = sget_kernel_info(base, "large_gemm_variant");
            if (tz_use_large_fused(d[0], d[1], d[2]) && !large.empty() &&
                get_kernel_info(base + "@" + large, "blocksize") != JSON_NOT_FOUND)
                key = base + "@" + large;
        }
    }
    int per_cu = get_kernel_info(key, "gridsize");
    int bs = get_kernel_info(key, "blocksize");
    int group = get_kernel_info(key, "group");
    if (per_cu == JSON_NOT_FOUND || bs == JSON_NOT_FOUND) logger.ERROR("kinfo has no entry for {" + key + "}");
    if (group == JSON_NOT_FOUND || group < 1) group = 1;
    int grid = launch_grid > 0 ? launch_grid : cuCount() * per_cu;
    // a workgroup-split kernel needs whole groups on every XCD
    const int quantum = 8 * group;
    if (grid % quantum) grid = (grid / quantum + 1) * quantum;
    if (launch_block > 0 && launch_block != bs)
        logger.ERROR("fused kernel {" + key + "} is built for " + std::to_string(bs) + " threads per workgroup");
    return new MixKernel(1, key, be, tz, dim3(grid, 1, 1), dim3(bs, 1, 1), be_start, be_end, tile_start, tile_end);
}

MixKernel *createBePairMix(GPTBKernel *first, GPTBKernel *second, int start1, int end1, int start2, int end2,
                           const std::string &variant, int launch_grid)
{
    const std::string base = first->kernelName + "_" + second->kernelName;
    const std::string key = variant.empty() ? base : base + "@" + variant;
    const int per_cu = get_kernel_info(key, "gridsize");
    const int bs = get_kernel_info(key, "blocksize");
    int group = get_kernel_info(key, "group");
    if (per_cu == JSON_NOT_FOUND || bs == JSON_NOT_FOUND) logger.ERROR("kinfo has no entry for {" + key + "}");
    if (group == JSON_NOT_FOUND || group < 1) group = 1;
    int grid = launch_grid > 0 ? launch_grid : cuCount() * per_cu;
    const int quantum = 8 * group;   // whole groups on every XCD
    if (grid % quantum) grid = (grid / quantum + 1) * quantum;
    return new MixKernel(2, key, first, second, dim3(grid, 1, 1), dim3(bs, 1, 1), start1, end1, start2, end2);
}

// "<a>_<b>" with a < b alphabetically (src/Creator.cu:341-816 lists its pairs one by one;
// here every pair of the four best-effort kernels exists): both kernels over their full
// ranges, memoised.
MixKernel *createMixKernel(const std::string &name)
{
    auto hit = mixKernelMap.find(name);
    if (hit != mixKernelMap.end()) return hit->second;
    const size_t cut = name.find('_');
    if (cut == std::string::npos || get_kernel_info(name, "blocksize") == JSON_NOT_FOUND)
        logger.ERROR("Creator: Mix kernel not found: " + name);
    GPTBKernel *first = createKernel(name.substr(0, cut));
    GPTBKernel *second = createKernel(name.substr(cut + 1));
    MixKernel *mix = createBePairMix(first, second, first->gptbParams.ptb_start_block_pos,
                                     first->gptbParams.ptb_end_block_pos, second->gptbParams.ptb_start_block_pos,
                                     second->gptbParams.ptb_end_block_pos, "", 0);
    mixKernelMap[name] = mix;
    return mix;
}
