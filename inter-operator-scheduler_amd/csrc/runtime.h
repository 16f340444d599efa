// Device-side half of the runtime: the process-wide device context (stream pool, reusable arena, options,
// kernel-configuration cache) and Session, a plan bound to device memory that can be run, timed per
// stage and profiled per operation.
#pragma once

#include <hip/hip_runtime.h>

#include <map>
#include <memory>
#include <string>
#include <vector>

#include "plan.h"
#include "fused.h"

namespace ios {

void hip_check(hipError_t status, const char *what, const char *file, int line);
#define IOS_HIP(call) ::ios::hip_check((call), #call, __FILE__, __LINE__)

// Streams: one HIP stream per group, event fork/join.  Fused: one launch per level of a multi-group stage
// (see fused.h).  The *Graph modes capture the same issue sequence into a hipGraph and replay it.
enum class ExecMode { Streams, Graph, Fused, FusedGraph };

class DeviceContext {
public:
    static DeviceContext &get();   // initialises the device on first use

    int num_cus() const { return num_cus_; }
    const std::string &name() const { return name_; }
    const std::string &arch() const { return arch_; }
    hipStream_t stream(int group) { return streams_[group]; }

    // a process-wide arena reused by the stateless latency / inference entry points
    float *shared_arena(size_t floats);
    void *shared_table(size_t bytes);   // companion buffer for the launch tables of such sessions

    void set_option(const std::string &key, const std::string &value);
    ExecMode exec_mode() const { return exec_mode_; }
    bool fused_executor() const { return exec_mode_ == ExecMode::Fused || exec_mode_ == ExecMode::FusedGraph; }
    bool autotune() const { return autotune_; }
    // split-K partial sums are added by a second kernel (Kernel), by the last block of a tile inside the convolution
    // kernel with the slices of a tile anywhere on the device (Inline), or the same with the slices of a tile numbered
    // onto one XCD, where they meet in that XCD's L2 (Xcd; the default when the placement probe at start-up found the
    // dispatcher's round-robin rule, and until a kernel reports a block somewhere else)
    enum class ReduceMode { Kernel, Inline, Xcd };
    ReduceMode reduce_mode() const { return reduce_mode_ == ReduceMode::Xcd && !xcd_usable_ ? ReduceMode::Inline : reduce_mode_; }
    bool inline_reduce() const { return reduce_mode_ != ReduceMode::Kernel; }
    // What the launchers take, for the mode in force and a launch on stream `group` of the pool.  The XCD a block lands
    // on depends on the stream (every stream starts its round-robin at an XCC of its own), so the XCD-local form needs
    // to know the stream; placement_known = false (kernels captured into a graph that forks: the replay runs them on
    // streams of its own) gives the device-wide form.
    SplitKReduce split_reduce(unsigned *counters, int group = 0, bool placement_known = true) const;
    // Throws when a kernel of the XCD-local form has reported a block on another XCC than the numbering assumes (results
    // of passes since the last check may be wrong); the form is switched off for the rest of the process first, so the
    // caller's next plan uses the device-wide form.
    void check_xcd_fault();
    bool xcd_usable() const { return xcd_usable_; }
    // testing aid: force one kernel configuration for every matrix-path convolution (-1 / 0 = off)
    int forced_variant() const { return forced_variant_; }
    int forced_split_k() const { return forced_split_k_; }
    std::string info_json() const;

    // Kernel configuration for a matrix-path convolution: the measured best when autotuning is on (cached
    // per problem signature for the life of the process, and in the file named by IOS_TUNE_CACHE when set),
    // else the closed-form model; the testing overrides win over both.
    // `share` = number of groups running concurrently with this convolution (1 = alone on the device).
    // allow_tuning = false never measures (measuring allocates scratch tensors): a shape that has no cached winner
    // gets the closed-form choice.
    ConvLaunch choose_launch(const ConvProblem &p, int share, bool allow_tuning = true);

    // Static device scratch of the entry point that allocates nothing: address on device 0 (resolved once, when the
    // context is created) and size in bytes.
    float *static_scratch() const { return static_scratch_; }
    static size_t static_scratch_bytes();
    static constexpr int kShareClasses = 4;   // footprint budgets 1, 1/2, 1/4, 1/8 of the device
    struct TunedConv {
        ConvLaunch best[kShareClasses];
    };
    std::map<std::string, TunedConv> tuned;

private:
    DeviceContext();
    TunedConv tune_conv(const ConvProblem &p);
    float *tuning_buffer(int which, size_t floats);
    unsigned *tuning_counters(size_t count);
    float *static_scratch_ = nullptr;
    unsigned *tune_counters_ = nullptr;
    size_t tune_counter_count_ = 0;
    ReduceMode reduce_mode_ = ReduceMode::Xcd;
    bool xcd_usable_ = false;       // the start-up probe found blocks with equal index % 8 on one XCC, launch after launch
    unsigned xcd_map_[kMaxGroups] = {};   // per stream of the pool: that XCC per index % 8, four bits each
    unsigned *xcd_fault_ = nullptr; // one word of pinned host memory the kernels can write
    void probe_xcd_placement();
    int precision_ = PREC_FP32;   // operand type of the matrix-path convolutions (reduced-precision modes: PREC_BF16, PREC_FP16)
    bool share_cost_rule_ = true;   // share classes weigh time by the held share of the device (false: hard footprint budgets)
    int share_threads_per_cu_ = 1024;   // resident threads per compute unit the share-class budgets assume (four wavefronts per SIMD)
    void load_tune_cache();
    std::string settings_token() const;
    float *tune_buf_[4] = {nullptr, nullptr, nullptr, nullptr};
    size_t tune_floats_[4] = {0, 0, 0, 0};
    std::string tune_cache_path_;
    int num_cus_ = 0;
    std::string name_, arch_;
    hipStream_t streams_[kMaxGroups];
    float *arena_ = nullptr;
    size_t arena_floats_ = 0;
    void *table_ = nullptr;
    size_t table_bytes_ = 0;
    // defaults: fused stage launches (stream fork / join costs more than the batch-1 kernels it would overlap) and
    // measured kernel configurations, like the reference's exhaustive algorithm search on first sight of a shape
    ExecMode exec_mode_ = ExecMode::Fused;
    bool autotune_ = true;
    int forced_variant_ = -1;
    int forced_split_k_ = 0;
};

class Session {
public:
    // Where a session's device memory comes from: its own allocation, the context's shared arena (one such session at
    // a time), or the static scratch array (one at a time; such a session allocates nothing, creates no events, and
    // issues every operator on the main stream in schedule order whatever the executor option says).
    enum class Storage { Own, Shared, Static };
    Session(Plan plan, Storage storage);
    Session(Plan plan, bool shared) : Session(std::move(plan), shared ? Storage::Shared : Storage::Own) {}
    ~Session();
    void release() noexcept;   // frees device memory, events and the captured graph; safe to call twice
    Session(const Session &) = delete;
    Session &operator=(const Session &) = delete;

    const Plan &plan() const { return plan_; }

    void set_input(const float *host);
    // returns false (and prints like the reference runtime) when no convolution has that name
    bool set_conv_weights(const char *name, const float *weight, const float *bias);
    void get_output(float *host);
    void get_tensor(const std::string &name, float *host);

    void run();   // one forward pass, synchronised
    void forward();       // one forward pass queued without waiting (stream launches or graph replay, by the execution mode)
    void synchronize();   // waits for everything queued
    // reference timing protocol for graphs / blocks: per repeat the mean of `number` individually
    // bracketed forward passes; optional per-stage times from events recorded after every stage
    void measure(int warmup, int number, int repeat, bool profile_stage, float *results, float *stage_results);
    // reference timing protocol for stage probes: `number` back-to-back passes in one bracket
    void measure_back_to_back(int warmup, int number, int repeat, float *results);
    void profile_ops(int warmup, int repeat, float *ms);
    // The kernel launches of one forward pass as the executor in force issues them (fused executors: one launch per
    // level of a multi-group stage, stand-alone kernels for single-group stages; stream executors: one per operation),
    // in issue order.
    struct LaunchRecord {
        int stage = 0;
        std::string kernel;      // e.g. "fused_kernel<512>", "conv_kernel<wq_m32n16_w8_t16>", "pool_kernel"
        std::vector<int> ops;    // indices into plan().ops
        int blocks = 0, threads = 0;
        int fused_level = -1;    // index into the stage's fused launches, -1 for a stand-alone kernel
    };
    std::vector<LaunchRecord> launches();
    std::string describe_launches();   // JSON array with the algorithmic flops and bytes of every launch
    // ms[i]: mean HIP-event time of launch i issued `repeat` times back to back on the launch stream
    void profile_launches(int warmup, int repeat, float *ms, int capacity);

private:
    void setup();
    void tune_convs();
    void launch_op(const PlanOp &op, int group);   // on stream `group` of the pool
    unsigned *counters_of(const PlanConv &c) const;
    const float *bias_of(const PlanConv &c) const { return base_ + (c.linear ? c.zero_bias_off : c.bias_off); }
    void enqueue(bool stage_events);   // issue one forward pass according to the execution mode
    void enqueue_streams(bool stage_events);
    void enqueue_fused(bool stage_events);
    void enqueue_serial();
    void build_fused();
    void build_graph();
    void copy_out(const ViewRef &view, float *host);
    TensorView tv(const ViewRef &v) const;

    Plan plan_;
    DeviceContext &ctx_;
    float *base_ = nullptr;
    bool owns_memory_ = false;
    bool static_ = false;
    std::vector<hipEvent_t> fork_events_;                 // per stage (multi-group stages only)
    std::vector<std::vector<hipEvent_t>> join_events_;    // per stage, per extra group
    std::vector<hipEvent_t> stage_events_;                // per stage, profile mode
    hipEvent_t start_ = nullptr, stop_ = nullptr;
    struct FusedLaunch {
        int threads, first_item, num_items, total_blocks, smem_bytes;
        int single_op;   // >= 0: no fused launch, this plan operation is launched with its stand-alone kernel
        FusedHeader header;
        std::vector<int> ops;   // plan operations behind the items (a two-kernel split-K reduction names its convolution)
    };
    std::vector<std::vector<FusedLaunch>> fused_stages_;   // per stage; empty for stages whose operations all follow each other
    void *fused_items_ = nullptr;                          // device copy of all work items
    std::vector<WorkItem> fused_items_host_;
    bool fused_built_ = false;
    bool capturing_forks_ = false;   // a graph capture of the stream executor is under way (the replay chooses the streams)
    hipGraph_t graph_ = nullptr;
    ExecMode graph_mode_ = ExecMode::Graph;                // mode the captured graph was built for
    hipGraphExec_t graph_exec_ = nullptr;
};

}  // namespace ios
