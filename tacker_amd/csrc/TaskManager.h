// TaskManager.h -- QoS-aware co-location of one latency-critical (LC) task with
// best-effort (BE) kernels (src/TaskManager.h of the reference).
//
// Same public surface: TaskManager(Task*, be1, be2), executeAllTasks(mode, stream),
// execute_with_one_cd_kernel(mode, stream), the free functions
// mixcudnnConvolutionForward / mixcublasSgemm / get_mnk_from_cudnn_args.  The
// decision arithmetic of the reference's hot loop (src/TaskManager.cu:586-640) is
// factored into QosPolicy so that it can be exercised with synthetic durations.
#pragma once

#include <string>
#include <vector>

#include "GPTBKernel.h"
#include "Task.h"

// {M, N, K} of the GEMM a convolution lowers to, from the 14 ints
// {n,c,h,w, k,c,kh,kw, pad_h,pad_w, stride_h,stride_w, dil_h,dil_w}
// (src/TaskManager.cu:92-123).
std::vector<int> get_mnk_from_cudnn_args(std::vector<int> &cudnn_args);

// One fused launch: the LC convolution's GEMM (after im2col) together with blocks
// [cd_start_blk, cd_end_blk) of the BE kernel (src/TaskManager.cu:125-306).
void mixcudnnConvolutionForward(std::vector<int> &cudnn_args, GPTBKernel *gptb_cd_kernel,
                                int cd_start_blk, int cd_end_blk, cudaStream_t stream);
// One fused launch: an LC fully-connected GEMM {m,n,k} + BE blocks (src/TaskManager.cu:309-400).
void mixcublasSgemm(std::vector<int> &gemm_args, GPTBKernel *gptb_cd_kernel, int cd_start_blk,
                    int cd_end_blk, cudaStream_t stream);

// The per-query accounting of the scheduler, free of any device call.
struct QosPolicy {
    float qos_budget_ms = 50.0f;   // per LC query (src/TaskManager.cu:571)
    float guard_ms = 4.0f;         // headroom guard band (:586)

    // BE blocks per 64x64 GEMM tile for a GEMM of depth K_GLOBAL: kinfo entry
    // "tzgemm_<be>"[K]; when absent, the K=4096 entry scaled linearly by K (:593-598).
    static float blockRatio(const std::string &be_name, int K_GLOBAL);
    // kinfo entry "tzgemm_<be>"["whole_kernel_gain"]: serial time / fused time measured with the
    // whole best-effort kernel in one fused launch; 1 when kinfo has none (the reference always
    // fuses, and credits a launch only if it beat the solo launches, :696-700)
    static float wholeKernelGain(const std::string &be_name);
    // the gain from which on Tacker mode lets the whole kernel ride: 3 % clear of breaking even
    static constexpr float kWholeKernelGainMin = 1.03f;
    // how many BE blocks ride along with a GEMM of `tiles` tiles (:599-600).  Tacker mode lets the
    // whole kernel ride unless kinfo says that this loses against the two launches
    // (wholeKernelGain < 1); it then carries the slice Aker mode would.
    static int coLocatedBlocks(ExecutionMode mode, const std::string &be_name, int tiles, int K_GLOBAL,
                               int be_total_blocks);
    // solo if the remaining budget cannot cover the rest of the query plus the guard (:586)
    bool mustRunSolo(float qos_headroom, float lc_time_remaining) const
    {
        return qos_headroom < lc_time_remaining + guard_ms;
    }
    struct Outcome {
        bool counted_as_mixed;   // the fused launch beat "LC alone then BE share alone"
        float charged_ms;        // what the query's budget is charged
        float earned_ms;         // time saved against serial execution (0 if not mixed)
    };
    // (:628-640) solo_lc_ms = profiled LC kernel time; be_ms = BE kernel's full solo time
    static Outcome account(unsigned mixable, float measured_ms, float solo_lc_ms, float be_ms,
                           int cd_blocks, int be_total_blocks);
};

struct TaskManagerReport {
    float lc_solo_ms = 0.0f;            // sum of profiled LC kernel times ("[PRE]")
    float be1_solo_ms = 0.0f, be2_solo_ms = 0.0f;
    long long be_blocks_executed = 0;   // BE blocks carried by fused launches in the last query
    int mix_times = 0, mixable_times = 0;
    int fusion_disabled = 0;            // LC kernels that ended the run barred from fusion
    float time_earned_ms = 0.0f;
    float qos_headroom_left_ms = 0.0f;
    float stage1_be_ms = 0.0f, stage2_be_ms = 0.0f;
    float be_mix_ms = 0.0f;             // fused launch of the two BE kernels (0 if the pair has no kernel)
    std::vector<float> query_latency_ms;   // one entry per co-located LC query
    std::vector<float> solo_latency_ms;    // one entry per solo LC query (profiling passes)
    // whole queries timed end to end (end_to_end_queries > 0): all launches of a query between one
    // pair of events, no synchronisation between kernels; and the same span on the host clock
    std::vector<float> e2e_colocated_ms, e2e_solo_ms;
    std::vector<float> e2e_colocated_wall_ms, e2e_solo_wall_ms;
    std::vector<float> e2e_graph_ms, e2e_graph_wall_ms;   // the solo query launched as one captured graph
};

class TaskManager {
public:
    TaskManager(Task *lc_task, const std::string &be_task1, const std::string &be_task2);
    ~TaskManager();
    void executeAllTasks(ExecutionMode mode, cudaStream_t stream);
    void execute_with_one_cd_kernel(ExecutionMode mode, cudaStream_t stream);

    Task *lc_task;
    std::string be_task1_name;
    std::string be_task2_name;
    int be_task_finish_num = 0;   // complete passes over the BE kernel's blocks

    // knobs the reference hard-codes
    QosPolicy policy;
    int warmup_queries = 5;
    int profile_queries = 10;
    int queries = 5;
    bool verbose = true;
    // Not in the reference: an LC kernel whose fused launch lost against "LC alone, then the
    // BE share alone" this many times in a row is launched alone from then on (Aker mode).
    // The static load ratios are measured on GEMMs that fill the GPU; layers with few tiles
    // can still lose, and every lost fusion stretches the LC query for nothing.  0 = never
    // stop (the reference's behaviour).
    int fusion_strikes_limit = 3;
    int fusion_retry_period = 64;   // queries between two chances for a barred kernel (0 = never again)
    // Not in the reference: before the co-located queries, measure for every mixable LC kernel
    // how many best-effort blocks its fused launch should carry (Aker mode), instead of taking
    // tiles x block_ratio(K) from kinfo.  That table is measured on GEMMs that fill the GPU; a
    // batch-1 layer with a few dozen tiles leaves most CUs free, and what those CUs can take
    // depends on the layer and on the best-effort kernel.  The fused launch is timed with
    // be_total / 256, / 128, ... blocks and the count with the largest earned time
    // (lc alone + share of be alone - fused) is kept among those whose fused launch stays
    // within (1 + calibrate_max_stretch) of the LC kernel alone; none -> the kernel runs alone.
    bool calibrate_blocks = false;
    float calibrate_max_stretch = 0.10f;
    std::vector<int> calibrated_blocks;   // per LC kernel, filled by the last calibrated run
    // > 0: the calibration pass chooses for the query as a whole -- per kernel at most one of the
    // timed (count, form) options, such that the sum of what the fused launches add to their
    // kernels stays within calibrate_query_stretch of the query's solo time and the earned time
    // is the largest possible; calibrate_max_stretch then only bounds what a single kernel may
    // be stretched by (and ends the ladder of counts for it).  0: the best count per kernel.
    float calibrate_query_stretch = 0.0f;
    int calibrate_passes = 3;             // timed fused launches per (kernel, count, form)
    // Forms of the fused kernel the calibration pass tries for every LC kernel ("" = the one kinfo
    // names for the pair); it keeps, per LC kernel, the form and count that earned most.  A short
    // layer can do better in a form with fewer best-effort waves per workgroup: the launch of a
    // 512-thread workgroup costs less than that of a 768-thread one.
    std::vector<std::string> calibrate_variants{""};
    std::vector<std::string> calibrated_variant;   // per LC kernel, beside calibrated_blocks
    // Not in the reference (its latency of a query is the sum of per-kernel intervals, each
    // followed by a synchronisation, src/TaskManager.cu:620-624): after the co-located queries,
    // run this many more queries of each kind -- every kernel alone, and with the best-effort
    // blocks the last co-located query carried -- with nothing between the launches of a query,
    // timed by one pair of events and by the host's steady clock around the query.  What a
    // client of the latency-critical service would see: launch gaps and host time included.
    int end_to_end_queries = 0;
    TaskManagerReport report;

private:
    void run(ExecutionMode mode, cudaStream_t stream, bool with_second_stage);
};
