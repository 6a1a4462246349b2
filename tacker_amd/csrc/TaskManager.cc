#include "TaskManager.h"

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdio>
#include <unordered_map>

#include "Creator.h"
#include "Logger.h"
#include "Recorder.h"
#include "json.h"
#include "tzgemm_kernel.h"
#include "dnn/vgg16.h"

extern Logger logger;
extern Recorder recorder;
extern std::unordered_map<std::string, void *> fmap;

// im2col staging buffers of the LC convolutions (src/TaskManager.cu:26-33); they
// grow on demand instead of being sized once.
static float *bottom = nullptr;
static float *col_buffer = nullptr;
static long long bottom_floats = 0, col_floats = 0;

static void ensure(float **p, long long *have, long long need)
{
    if (need <= *have) return;
    TK_SAFE_CALL(tkDeviceSynchronize());
    if (*p) TK_SAFE_CALL(tkFree(*p));
    TK_SAFE_CALL(tkMalloc((void **)p, (size_t)need * sizeof(float)));
    TK_SAFE_CALL(tkMemset(*p, 0, (size_t)need * sizeof(float)));
    *have = need;
}

std::vector<int> get_mnk_from_cudnn_args(std::vector<int> &a)
{
    const int height_col = (a[2] + 2 * a[8] - (a[12] * (a[6] - 1) + 1)) / a[10] + 1;
    const int width_col = (a[3] + 2 * a[9] - (a[13] * (a[7] - 1) + 1)) / a[11] + 1;
    return std::vector<int>{a[0] * height_col * width_col, a[4], a[6] * a[7] * a[1]};
}

// im2col of the convolution's input on `stream`, then the shapes of its GEMM
static std::vector<int> lowerConvolution(std::vector<int> &a, cudaStream_t stream)
{
    int input_n = a[0], input_c = a[1], input_h = a[2], input_w = a[3];
    int kernel_h = a[6], kernel_w = a[7], pad_h = a[8], pad_w = a[9];
    int stride_h = a[10], stride_w = a[11], dilation_h = a[12], dilation_w = a[13];
    int height_col = (input_h + 2 * pad_h - (dilation_h * (kernel_h - 1) + 1)) / stride_h + 1;
    int width_col = (input_w + 2 * pad_w - (dilation_w * (kernel_w - 1) + 1)) / stride_w + 1;
    int num_kernels = input_n * input_c * height_col * width_col;
    int im_size = input_n * input_c * input_h * input_w;
    int col_size = num_kernels * kernel_h * kernel_w;
    ensure(&bottom, &bottom_floats, im_size);
    ensure(&col_buffer, &col_floats, col_size);
    void *args[] = {&num_kernels, &bottom, &input_h, &input_w, &kernel_h, &kernel_w, &pad_h, &pad_w,
                    &stride_h, &stride_w, &dilation_h, &dilation_w, &height_col, &width_col, &col_buffer,
                    &im_size, &col_size};
    TK_SAFE_CALL(tkLaunchKernel(fmap.at("im2col"), dim3(cuCount() * 2).raw(), dim3(256).raw(), args, 0, stream));
    return get_mnk_from_cudnn_args(a);
}

static void launchMixedGemm(int M_INPUT, int N_INPUT, int K_INPUT, GPTBKernel *gptb_cd_kernel,
                            int cd_start_blk, int cd_end_blk, cudaStream_t stream)
{
    const std::vector<int> d = getTZGEMMGridDim(M_INPUT, N_INPUT, K_INPUT);
    OriTZGEMMKernel ori_tzgemm(0, d[0], d[1], d[2]);
    GPTBKernel gptb_tzgemm_kernel(1, "tzgemm", "gptb_tzgemm", &ori_tzgemm, dim3(cuCount(), 1, 1),
                                  dim3(TZ_THREADS, 1, 1), 0, d[3]);
    if (cd_end_blk <= cd_start_blk) {   // nothing to co-locate: the GEMM alone
        gptb_tzgemm_kernel.execute(stream);
        return;
    }
    MixKernel *mix = createTzgemmMix(gptb_cd_kernel, &gptb_tzgemm_kernel, cd_start_blk, cd_end_blk, 0, d[3], "", 0, 0);
    mix->execute(stream);
    delete mix;   // the launch has copied its arguments
}

void mixcudnnConvolutionForward(std::vector<int> &cudnn_args, GPTBKernel *gptb_cd_kernel, int cd_start_blk,
                                int cd_end_blk, cudaStream_t stream)
{
    const std::vector<int> mnk = lowerConvolution(cudnn_args, stream);
    launchMixedGemm(mnk[0], mnk[1], mnk[2], gptb_cd_kernel, cd_start_blk, cd_end_blk, stream);
}

void mixcublasSgemm(std::vector<int> &gemm_args, GPTBKernel *gptb_cd_kernel, int cd_start_blk,
                    int cd_end_blk, cudaStream_t stream)
{
    launchMixedGemm(gemm_args[0], gemm_args[1], gemm_args[2], gptb_cd_kernel, cd_start_blk, cd_end_blk, stream);
}

// ---------------------------------------------------------------------------- policy

float QosPolicy::blockRatio(const std::string &be_name, int K_GLOBAL)
{
    float block_ratio = fget_kernel_info("tzgemm_" + be_name, std::to_string(K_GLOBAL));
    if (block_ratio == JSON_NOT_FOUND) {
        const float base_block_ratio = fget_kernel_info("tzgemm_" + be_name, std::to_string(4096));
        block_ratio = base_block_ratio * K_GLOBAL / 4096;
    }
    return block_ratio;
}

float QosPolicy::wholeKernelGain(const std::string &be_name)
{
    const float gain = fget_kernel_info("tzgemm_" + be_name, "whole_kernel_gain");
    return gain == JSON_NOT_FOUND ? 1.0f : gain;
}

int QosPolicy::coLocatedBlocks(ExecutionMode mode, const std::string &be_name, int tiles, int K_GLOBAL,
                               int be_total_blocks)
{
    // the whole BE kernel rides along, unless it is known to lose that way
    if (mode == ExecutionMode::Tacker && wholeKernelGain(be_name) >= kWholeKernelGainMin) return be_total_blocks;
    return std::min(int(tiles * blockRatio(be_name, K_GLOBAL)), be_total_blocks);
}

QosPolicy::Outcome QosPolicy::account(unsigned mixable, float measured_ms, float solo_lc_ms, float be_ms,
                                      int cd_blocks, int be_total_blocks)
{
    Outcome o{false, solo_lc_ms, 0.0f};
    if (mixable == 0) return o;
    const float serial_ms = solo_lc_ms + be_ms * cd_blocks / be_total_blocks;
    if (measured_ms > serial_ms) return o;   // fusing did not pay: charge the solo time
    o.counted_as_mixed = true;
    o.charged_ms = measured_ms;
    o.earned_ms = serial_ms - measured_ms;
    return o;
}

// ---------------------------------------------------------------------------- manager

TaskManager::TaskManager(Task *lc_task, const std::string &be_task1, const std::string &be_task2)
    : lc_task(lc_task), be_task1_name(be_task1), be_task2_name(be_task2)
{
}

TaskManager::~TaskManager() {}

namespace {
struct Stopwatch {
    tkEvent_t a = nullptr, b = nullptr;
    Stopwatch()
    {
        TK_SAFE_CALL(tkEventCreate(&a));
        TK_SAFE_CALL(tkEventCreate(&b));
    }
    ~Stopwatch()
    {
        tkEventDestroy(a);
        tkEventDestroy(b);
    }
    void start(cudaStream_t s) { TK_SAFE_CALL(tkEventRecord(a, s)); }
    float stop(cudaStream_t s)
    {
        float ms = 0.0f;
        TK_SAFE_CALL(tkEventRecord(b, s));
        TK_SAFE_CALL(tkEventSynchronize(b));
        TK_SAFE_CALL(tkEventElapsedTime(&ms, a, b));
        return ms;
    }
};
}  // namespace

void TaskManager::executeAllTasks(ExecutionMode mode, cudaStream_t stream) { run(mode, stream, true); }
void TaskManager::execute_with_one_cd_kernel(ExecutionMode mode, cudaStream_t stream) { run(mode, stream, false); }

void TaskManager::run(ExecutionMode mode, cudaStream_t stream, bool with_second_stage)
{
    Stopwatch watch;
    report = TaskManagerReport();
    const size_t nk = lc_task->kernels.size();

    for (int i = 0; i < warmup_queries; ++i) {
        lc_task->initExecution();
        for (auto &lc_kernel : lc_task->kernels) lc_kernel->execute(stream);
    }
    TK_SAFE_CALL(tkDeviceSynchronize());

    GPTBKernel *be_kernel1 = createKernel(be_task1_name);
    const int be_total = be_kernel1->gptbParams.ptb_end_block_pos;

    // duration predictor, input 1: mean solo time of every LC kernel
    std::vector<float> lc_kernel_time_vec(nk, 0.0f);
    for (int i = 0; i < profile_queries; ++i) {
        lc_task->initExecution();
        float query_ms = 0.0f;
        for (size_t idx = 0; idx < nk; ++idx) {
            Kernel *lc_kernel = lc_task->kernels[idx];
            if (!i && lc_kernel->mixable != 0) report.mixable_times++;
            if (lc_kernel->mixable == 1 && lc_kernel->getArgs().size() != 3)
                logger.ERROR("lc kernel: " + lc_kernel->kernelName + " mnk size is not 3");
            if (lc_kernel->mixable == 2 && lc_kernel->getArgs().size() != 14)
                logger.ERROR("lc kernel: " + lc_kernel->kernelName + " cudnn args size is not 14");
            watch.start(stream);
            lc_kernel->execute(stream);
            const float ms = watch.stop(stream);
            lc_kernel_time_vec[idx] += ms;
            query_ms += ms;
        }
        report.solo_latency_ms.push_back(query_ms);
    }
    for (auto &t : lc_kernel_time_vec) {
        t /= std::max(profile_queries, 1);
        report.lc_solo_ms += t;
    }
    if (verbose) printf("\n[PRE]lc kernel took %f ms to execute.\n", report.lc_solo_ms);
    // time still needed to finish the query from kernel i on
    std::vector<float> lc_headroom_vec(lc_kernel_time_vec);
    for (int i = (int)nk - 2; i >= 0; --i) lc_headroom_vec[i] += lc_headroom_vec[i + 1];

    // duration predictor, input 2: solo time of the BE kernels (time of n blocks = t * n / N)
    GPTBKernel *be_task1 = createKernel(be_task1_name);
    GPTBKernel *be_task2 = with_second_stage ? createKernel(be_task2_name) : nullptr;
    for (int i = 0; i < 10; ++i) {
        be_task1->execute(stream);
        if (be_task2) be_task2->execute(stream);
    }
    TK_SAFE_CALL(tkDeviceSynchronize());
    // mean of a few back-to-back launches: one launch alone right after a synchronisation is
    // timed with the start-up of the queue in it, and this figure prices every co-located block
    const int be_samples = 10;
    watch.start(stream);
    for (int i = 0; i < be_samples; ++i) be_task1->execute(stream);
    report.be1_solo_ms = watch.stop(stream) / be_samples;
    if (be_task2) {
        watch.start(stream);
        for (int i = 0; i < be_samples; ++i) be_task2->execute(stream);
        report.be2_solo_ms = watch.stop(stream) / be_samples;
    }

    // launch of LC kernel idx fused with BE blocks [from, to) of be_kernel1
    auto launch_mixed = [&](Kernel *lc_kernel, int from, int to, const std::string &variant = std::string()) {
        std::vector<int> args = lc_kernel->getArgs();
        std::vector<int> mnk = lc_kernel->mixable == 1 ? args : get_mnk_from_cudnn_args(args);
        if (auto *layer = dynamic_cast<LcGemmKernel *>(lc_kernel))
            layer->executeMixed(be_kernel1, from, to, stream, variant);   // the layer's own operands
        else if (lc_kernel->mixable == 1) mixcublasSgemm(mnk, be_kernel1, from, to, stream);
        else mixcudnnConvolutionForward(args, be_kernel1, from, to, stream);
    };

    // optional: measured block count per LC kernel instead of the kinfo table
    calibrated_blocks.clear();
    calibrated_variant.clear();
    if (calibrate_blocks && mode == ExecutionMode::Aker && be_total > 0) {
        calibrated_blocks.assign(nk, 0);
        calibrated_variant.assign(nk, "");
        std::vector<float> best_earned(nk, 0.0f);
        const int first = be_kernel1->gptbParams.ptb_start_block_pos;
        // every fused launch that was timed and kept its kernel within the per-kernel limit
        struct Option { int n; std::string form; float cost_ms, earned_ms; };
        std::vector<std::vector<Option>> options(nk);
        std::vector<std::string> forms;
        for (const std::string &v : calibrate_variants)
            if (v.empty() || get_kernel_info("tzgemm_" + be_task1_name + "@" + v, "blocksize") != JSON_NOT_FOUND)
                forms.push_back(v);
        if (forms.empty()) forms.push_back("");
        // the slices move through the best-effort kernel as they will in the co-located queries:
        // a slice that was launched a moment ago is served from the caches and looks cheaper
        int cal_cursor = first;
        for (const std::string &form : forms) {
            std::vector<bool> over(nk, false);   // a smaller count already stretched this kernel too far
            for (int divisor = 256; divisor >= 1; divisor /= 2) {
                const int n = std::max(1, be_total / divisor);
                std::vector<float> fused_ms(nk, 0.0f);
                const int timed = std::max(calibrate_passes, 1);
                for (int pass = -1; pass < timed; ++pass) {   // pass -1 warms up
                    lc_task->initExecution();
                    for (size_t idx = 0; idx < nk; ++idx) {
                        Kernel *lc_kernel = lc_task->kernels[idx];
                        if (lc_kernel->mixable == 0 || over[idx]) {
                            lc_kernel->execute(stream);
                            continue;
                        }
                        if (cal_cursor + n > be_total) cal_cursor = first;
                        const int from = cal_cursor, to = std::min(cal_cursor + n, be_total);
                        cal_cursor = to;
                        watch.start(stream);
                        launch_mixed(lc_kernel, from, to, form);
                        const float ms = watch.stop(stream);
                        if (pass >= 0) fused_ms[idx] += ms / timed;
                    }
                }
                for (size_t idx = 0; idx < nk; ++idx) {
                    if (lc_task->kernels[idx]->mixable == 0 || over[idx]) continue;
                    const float alone = lc_kernel_time_vec[idx];
                    if (fused_ms[idx] > (1.0f + calibrate_max_stretch) * alone) {
                        over[idx] = true;
                        continue;
                    }
                    const float earned = alone + report.be1_solo_ms * n / be_total - fused_ms[idx];
                    if (earned > 0.0f)
                        options[idx].push_back({n, form, std::max(fused_ms[idx] - alone, 0.0f), earned});
                    if (earned > best_earned[idx]) {
                        best_earned[idx] = earned;
                        calibrated_blocks[idx] = n;
                        calibrated_variant[idx] = form;
                    }
                }
            }
        }
        if (calibrate_query_stretch > 0.0f) {
            // A budget for the whole query instead of the best count per kernel: the launches to
            // fuse, one option per kernel at most, that earn most while the query grows by at most
            // calibrate_query_stretch of its solo time.  A short layer that earns a microsecond for
            // five of latency then leaves its share of the budget to a layer that earns four for one.
            // Exact by dynamic programming over the budget in steps of a thousandth.
            const int steps = 1000;
            const float budget_ms = calibrate_query_stretch * report.lc_solo_ms;
            // an option's cost in steps of the budget (steps + 1: does not fit)
            auto cost_steps = [&](const Option &opt) {
                if (budget_ms <= 0.0f) return opt.cost_ms > 0.0f ? steps + 1 : 0;
                return (int)std::min(std::ceil(opt.cost_ms / budget_ms * steps), (float)(steps + 1));
            };
            std::vector<float> best(steps + 1, 0.0f);
            std::vector<std::vector<int>> pick(nk, std::vector<int>(steps + 1, -1));
            for (size_t idx = 0; idx < nk; ++idx) {
                std::vector<float> next(best);
                for (size_t o = 0; o < options[idx].size(); ++o) {
                    const Option &opt = options[idx][o];
                    const int c = cost_steps(opt);
                    for (int u = c; u <= steps; ++u)
                        if (best[u - c] + opt.earned_ms > next[u]) {
                            next[u] = best[u - c] + opt.earned_ms;
                            pick[idx][u] = (int)o;
                        }
                }
                best.swap(next);
            }
            int u = steps;
            for (int idx = (int)nk - 1; idx >= 0; --idx) {
                const int o = pick[idx][u];
                calibrated_blocks[idx] = 0;
                calibrated_variant[idx] = "";
                best_earned[idx] = 0.0f;
                if (o < 0) continue;
                // pick[idx][u] was set while kernel idx was added on top of the state of the kernels
                // before it: walk back through that state
                const Option &opt = options[idx][(size_t)o];
                calibrated_blocks[idx] = opt.n;
                calibrated_variant[idx] = opt.form;
                best_earned[idx] = opt.earned_ms;
                u -= cost_steps(opt);
            }
        }
        if (verbose)
            for (size_t idx = 0; idx < nk; ++idx)
                if (lc_task->kernels[idx]->mixable != 0)
                    printf("[CAL] %s: %d blocks%s%s, earns %f ms\n", lc_task->kernels[idx]->kernelName.c_str(),
                           calibrated_blocks[idx], calibrated_variant[idx].empty() ? "" : " in form ",
                           calibrated_variant[idx].c_str(), best_earned[idx]);
    }

    // co-located queries: a cursor walks the BE kernel's blocks across launches
    int be_cursor = be_kernel1->gptbParams.ptb_start_block_pos;
    float qos_headroom = policy.qos_budget_ms;
    std::vector<int> strikes(nk, 0);   // consecutive fused launches of kernel i that did not pay
    std::vector<int> carried(nk, 0);   // best-effort blocks kernel i's launch carried in the last query
    for (int q = 0; q < queries; ++q) {
        lc_task->initExecution();
        qos_headroom = policy.qos_budget_ms;
        // a barred kernel gets one more chance every fusion_retry_period queries; kernel i takes
        // its chance in the queries congruent to i, so that the retries (each a launch expected
        // to lose) are spread over queries instead of piling up in one slow query
        if (fusion_retry_period > 0 && q >= fusion_retry_period)
            for (size_t idx = 0; idx < nk; ++idx)
                if (q % fusion_retry_period == (int)(idx % (size_t)fusion_retry_period))
                    strikes[idx] = std::min(strikes[idx], std::max(fusion_strikes_limit - 1, 0));
        long long cd_block_num_executed = 0;
        report.mix_times = 0;
        report.time_earned_ms = 0.0f;
        float query_ms = 0.0f;
        for (size_t idx = 0; idx < nk; ++idx) {
            Kernel *lc_kernel = lc_task->kernels[idx];
            int cd_block_num = 0;
            watch.start(stream);
            const bool barred = mode == ExecutionMode::Aker && fusion_strikes_limit > 0 &&
                                strikes[idx] >= fusion_strikes_limit;
            const bool calibrated = !calibrated_blocks.empty();
            if (policy.mustRunSolo(qos_headroom, lc_headroom_vec[idx]) || lc_kernel->mixable == 0 || barred ||
                (calibrated && calibrated_blocks[idx] == 0)) {
                lc_kernel->execute(stream);
            } else {
                if (calibrated) {
                    cd_block_num = calibrated_blocks[idx];
                } else {
                    std::vector<int> args = lc_kernel->getArgs();
                    std::vector<int> mnk = lc_kernel->mixable == 1 ? args : get_mnk_from_cudnn_args(args);
                    if (auto *layer = dynamic_cast<LcGemmKernel *>(lc_kernel)) mnk = layer->gemmDims();
                    const std::vector<int> MNKD = getTZGEMMGridDim(mnk[0], mnk[1], mnk[2]);
                    cd_block_num = QosPolicy::coLocatedBlocks(mode, be_task1_name, MNKD[3], MNKD[2], be_total);
                }
                const int end = std::min(be_cursor + cd_block_num, be_total);
                cd_block_num = end - be_cursor;
                launch_mixed(lc_kernel, be_cursor, end, calibrated ? calibrated_variant[idx] : std::string());
                be_cursor = end;
                if (be_cursor >= be_total) {   // one pass over the BE kernel done
                    be_cursor = be_kernel1->gptbParams.ptb_start_block_pos;
                    be_task_finish_num++;
                }
            }
            const float duration = watch.stop(stream);
            query_ms += duration;
            carried[idx] = cd_block_num;
            const unsigned mixed = cd_block_num > 0 ? lc_kernel->mixable : 0u;
            const QosPolicy::Outcome o = QosPolicy::account(mixed, duration, lc_kernel_time_vec[idx],
                                                            report.be1_solo_ms, cd_block_num, be_total);
            qos_headroom -= o.charged_ms;
            if (mixed) strikes[idx] = o.counted_as_mixed ? 0 : strikes[idx] + 1;
            if (o.counted_as_mixed) {
                cd_block_num_executed += cd_block_num;
                report.mix_times++;
                report.time_earned_ms += o.earned_ms;
            }
        }
        report.be_blocks_executed = cd_block_num_executed;
        report.query_latency_ms.push_back(query_ms);
    }
    // whole queries end to end, nothing between their launches: every kernel alone, then with what
    // the last co-located query carried (the cursor keeps walking the best-effort kernel's blocks)
    for (int kind = 0; kind < 2 && end_to_end_queries > 0; ++kind) {
        std::vector<float> &by_event = kind ? report.e2e_colocated_ms : report.e2e_solo_ms;
        std::vector<float> &by_clock = kind ? report.e2e_colocated_wall_ms : report.e2e_solo_wall_ms;
        for (int q = -2; q < end_to_end_queries; ++q) {   // two untimed queries first
            lc_task->initExecution();
            TK_SAFE_CALL(tkStreamSynchronize(stream));
            const auto t0 = std::chrono::steady_clock::now();
            watch.start(stream);
            for (size_t idx = 0; idx < nk; ++idx) {
                Kernel *lc_kernel = lc_task->kernels[idx];
                if (kind == 0 || carried[idx] <= 0 || lc_kernel->mixable == 0) {
                    lc_kernel->execute(stream);
                    continue;
                }
                const int end = std::min(be_cursor + carried[idx], be_total);
                launch_mixed(lc_kernel, be_cursor, end,
                             calibrated_variant.empty() ? std::string() : calibrated_variant[idx]);
                be_cursor = end >= be_total ? be_kernel1->gptbParams.ptb_start_block_pos : end;
            }
            const float ms = watch.stop(stream);   // waits for the query's last kernel
            const float wall = std::chrono::duration<float, std::milli>(std::chrono::steady_clock::now() - t0).count();
            if (q >= 0) {
                by_event.push_back(ms);
                by_clock.push_back(wall);
            }
        }
    }
    // ... and the query alone as one graph: its launches are the same every time, so they are recorded once
    // from a stream of their own and launched as a whole, which takes the host's per-launch cost out
    // of the query (a batch-1 query is bound by the host's launch rate otherwise)
    if (end_to_end_queries > 0) {
        cudaStream_t capture_stream = nullptr;
        tkGraphExec_t graph = nullptr;
        TK_SAFE_CALL(tkStreamCreate(&capture_stream));
        TK_SAFE_CALL(tkDeviceSynchronize());
        try {
            graph = lc_task->captureQuery(capture_stream);
        } catch (...) {
            tkStreamDestroy(capture_stream);
            throw;
        }
        for (int q = -2; q < end_to_end_queries; ++q) {
            lc_task->initExecution();
            TK_SAFE_CALL(tkStreamSynchronize(capture_stream));
            const auto t0 = std::chrono::steady_clock::now();
            watch.start(capture_stream);
            TK_SAFE_CALL(tkGraphLaunch(graph, capture_stream));
            const float ms = watch.stop(capture_stream);
            const float wall = std::chrono::duration<float, std::milli>(std::chrono::steady_clock::now() - t0).count();
            if (q >= 0) {
                report.e2e_graph_ms.push_back(ms);
                report.e2e_graph_wall_ms.push_back(wall);
            }
        }
        TK_SAFE_CALL(tkGraphExecDestroy(graph));
        TK_SAFE_CALL(tkStreamDestroy(capture_stream));
    }
    report.qos_headroom_left_ms = qos_headroom;
    report.fusion_disabled = 0;
    if (fusion_strikes_limit > 0)
        for (int v : strikes) report.fusion_disabled += v >= fusion_strikes_limit;
    report.stage1_be_ms = report.be_blocks_executed * report.be1_solo_ms / std::max(be_total, 1);
    if (verbose) {
        printf("execed be blks: %lld, mix times: %d/%d, time earned: %f\n", report.be_blocks_executed,
               report.mix_times, report.mixable_times, report.time_earned_ms);
        printf("[Ori] be_task1: %s, be_task2: %s\n", be_task1_name.c_str(), be_task2_name.c_str());
        printf("[Ori] BE task1 + task2 took %f + %f = %f ms to execute.\n", report.be1_solo_ms,
               report.be2_solo_ms, report.be1_solo_ms + report.be2_solo_ms);
    }

    // stage 2: the budget left after the LC query runs the two BE kernels fused
    // (src/TaskManager.cu:676-702): time the pair's fused launch; if it beats the two solo
    // launches the leftover budget is worth that much more BE work
    report.stage2_be_ms = std::max(0.0f, qos_headroom);
    report.be_mix_ms = 0.0f;
    if (be_task2 && be_task1_name != be_task2_name) {
        const std::string mix_be_name = be_task1_name < be_task2_name ? be_task1_name + "_" + be_task2_name
                                                                      : be_task2_name + "_" + be_task1_name;
        if (get_kernel_info(mix_be_name, "blocksize") != JSON_NOT_FOUND) {
            MixKernel *be_mix = createMixKernel(mix_be_name);
            for (int i = 0; i < 5; ++i) be_mix->execute(stream);
            TK_SAFE_CALL(tkDeviceSynchronize());
            watch.start(stream);   // timed the way the two kernels alone were
            for (int i = 0; i < be_samples; ++i) be_mix->execute(stream);
            const float mix_be_time = watch.stop(stream) / be_samples;
            report.be_mix_ms = mix_be_time;
            if (verbose) printf("[Mix] BE task1 + task2 took %f ms to execute.\n", mix_be_time);
            const float solo_sum = report.be1_solo_ms + report.be2_solo_ms;
            if (mode == ExecutionMode::Aker && mix_be_time > 0.0f && mix_be_time < solo_sum)
                report.stage2_be_ms = std::max(0.0f, qos_headroom * solo_sum / mix_be_time);
        }
    }
    if (verbose) {
        const char *who = mode == ExecutionMode::Aker ? "Aker" : "Tacker";
        printf("[Result] %s BE task took %f + %f(%f) = %f ms to execute.\n", who, report.stage1_be_ms,
               report.stage2_be_ms, qos_headroom, report.stage1_be_ms + report.stage2_be_ms);
    }
}
