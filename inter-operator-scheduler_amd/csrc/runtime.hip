// Stage executor, timers and device context.
//
// A forward pass walks the plan's stages.  Fused executor (default): a multi-group stage is issued as one
// fused launch per chain position on the main stream (see build_fused).  Streams executor: group g of a stage
// is issued to stream g of a fixed pool; stream 0 is the main stream; a multi-group stage forks (the extra
// streams wait on an event recorded on the main stream) and joins (the main stream waits on one event per
// extra stream).  Either way stage boundaries are device-side dependencies and the host never blocks inside
// a pass.  The graph modes capture the same issue sequence once into a hipGraph and replay it.
//
// Timing follows the reference runtime (src/ios/ios_runtime.cu:1328-1455): graph / block latency is the
// mean over `number` individually bracketed passes per repeat, with optional per-stage times from events
// recorded on the main stream after every stage; stage probes time `number` back-to-back passes inside
// one event pair.
#include "runtime.h"

#include "fused.h"

#include <algorithm>
#include <cstdio>
#include <cstring>
#include <sstream>
#include <stdexcept>

namespace ios {

void hip_check(hipError_t status, const char *what, const char *file, int line) {
    if (status == hipSuccess) return;
    std::ostringstream os;
    os << "HIP failure " << hipGetErrorString(status) << " (" << (int)status << ") in " << what << " at " << file << ":" << line;
    throw std::runtime_error(os.str());
}

// ---- static scratch ----------------------------------------------------------------------------------------------
// Device memory of graph_inference_no_alloc: a session created with Storage::Static lays its whole arena (operator
// outputs, filters, packed filters, split-K partial tiles and ticket counters) out in this array instead of
// allocating.  The device holds it from the moment the library is loaded until the process ends.  In host code
// the array's name is only a handle for hipGetSymbolAddress; kernels and copies get the address resolved below.
constexpr size_t kStaticScratchBytes = size_t(256) << 20;
static __device__ __align__(256) float scratch[kStaticScratchBytes / sizeof(float)];

size_t DeviceContext::static_scratch_bytes() { return kStaticScratchBytes; }

// ---- device context --------------------------------------------------------------------------------------------
DeviceContext &DeviceContext::get() {
    static DeviceContext instance;
    return instance;
}

DeviceContext::DeviceContext() {
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count < 1) throw std::runtime_error("no HIP device available");
    IOS_HIP(hipSetDevice(0));
    hipDeviceProp_t prop;
    IOS_HIP(hipGetDeviceProperties(&prop, 0));
    num_cus_ = prop.multiProcessorCount;
    name_ = prop.name;
    arch_ = prop.gcnArchName;
    for (int i = 0; i < kMaxGroups; i++) IOS_HIP(hipStreamCreateWithFlags(&streams_[i], hipStreamNonBlocking));
    // the library runs on device 0 only, which is current here: its copy of the array is the one ever used
    IOS_HIP(hipGetSymbolAddress(reinterpret_cast<void **>(&static_scratch_), HIP_SYMBOL(scratch)));
    probe_xcd_placement();
    const char *mode = getenv("IOS_EXECUTOR");
    if (mode != nullptr) set_option("executor", mode);
    const char *tune = getenv("IOS_AUTOTUNE");
    if (tune != nullptr) set_option("autotune", tune);
    const char *cache = getenv("IOS_TUNE_CACHE");
    if (cache != nullptr && cache[0] != '\0') {
        tune_cache_path_ = cache;
        load_tune_cache();
    }
}

// ---- placement of workgroups on XCDs --------------------------------------------------------------------------------
// The XCD-local split-K relies on blocks with equal index % 8 running on one XCD (the dispatcher deals the workgroups of
// a launch round-robin).  The rule is checked here, on launches of several sizes, before anything uses it, and every block
// of such a launch checks its own XCC id again (xcd_enter).
__global__ void xcc_probe_kernel(unsigned *out) {
    if (threadIdx.x == 0) out[blockIdx.x] = xcc_id();
}

void DeviceContext::probe_xcd_placement() {
    xcd_usable_ = false;
    if (hipHostMalloc(reinterpret_cast<void **>(&xcd_fault_), 64, hipHostMallocMapped) != hipSuccess || xcd_fault_ == nullptr) {
        xcd_fault_ = nullptr;
        (void)hipGetLastError();
        return;
    }
    *xcd_fault_ = 0;
    constexpr int kMost = 1031;
    unsigned *device = nullptr;
    IOS_HIP(hipMalloc(reinterpret_cast<void **>(&device), kMost * sizeof(unsigned)));
    std::vector<unsigned> host(kMost);
    bool consistent = true;
    // Measured on MI355X: inside a launch, block b runs on XCC (first + b) % 8, and `first` is a constant of the stream
    // the launch goes to (launch after launch, alone or beside launches of other streams, also for the nodes that a
    // captured graph runs on the stream it is launched on).
    for (int g = 0; g < kMaxGroups; g++) {
        int seen[8] = {-1, -1, -1, -1, -1, -1, -1, -1};
        for (int blocks : {kMost, 8, 250}) {
            for (int threads : {64, 512}) {
                hipLaunchKernelGGL(xcc_probe_kernel, dim3(blocks), dim3(threads), 0, streams_[g], device);
                IOS_HIP(hipMemcpyAsync(host.data(), device, blocks * sizeof(unsigned), hipMemcpyDeviceToHost, streams_[g]));
                IOS_HIP(hipStreamSynchronize(streams_[g]));
                for (int b = 0; b < blocks; b++) {
                    if (seen[b & 7] < 0) seen[b & 7] = (int)host[b];
                    consistent = consistent && seen[b & 7] == (int)host[b] && host[b] < 16;
                }
            }
        }
        xcd_map_[g] = 0;
        for (int c = 0; c < 8; c++) xcd_map_[g] |= (unsigned)(seen[c] & 15) << (4 * c);
    }
    IOS_HIP(hipFree(device));
    xcd_usable_ = consistent;
}

SplitKReduce DeviceContext::split_reduce(unsigned *counters, int group, bool placement_known) const {
    SplitKReduce r;
    r.counters = inline_reduce() ? counters : nullptr;
    r.xcd_local = reduce_mode() == ReduceMode::Xcd && placement_known && group >= 0 && group < kMaxGroups;
    r.xcd_map = r.xcd_local ? xcd_map_[group] : 0;
    r.fault = xcd_fault_;
    return r;
}

void DeviceContext::check_xcd_fault() {
    if (xcd_fault_ == nullptr || *reinterpret_cast<volatile unsigned *>(xcd_fault_) == 0) return;
    *xcd_fault_ = 0;
    xcd_usable_ = false;
    tuned.clear();
    throw std::runtime_error("a split-K convolution found a workgroup on another XCD than the round-robin placement it relies on: results since the "
                             "last synchronisation may be wrong.  The XCD-local form is switched off for the rest of this process; create the session again");
}

// ---- kernel configuration choice ----------------------------------------------------------------------------------
static std::string conv_signature(const ConvProblem &p) {
    std::ostringstream os;
    os << p.B << ' ' << p.IC << ' ' << p.H << ' ' << p.W << ' ' << p.OC << ' ' << p.KH << ' ' << p.KW << ' ' << p.sh << ' ' << p.sw
       << ' ' << p.ph << ' ' << p.pw << ' ' << p.groups;
    return os.str();
}

// the measured winners of the share classes depend on these settings: they are part of every cache key
std::string DeviceContext::settings_token() const {
    std::ostringstream os;
    os << (share_cost_rule_ ? "cost" : "budget") << '/' << share_threads_per_cu_ << '/'
       << (reduce_mode() == ReduceMode::Xcd ? "xcd" : reduce_mode() == ReduceMode::Inline ? "inline" : "kernel")
       << (fused_executor() ? "" : "/own-launches");
    return os.str();
}

void DeviceContext::load_tune_cache() {
    FILE *f = fopen(tune_cache_path_.c_str(), "r");
    if (f == nullptr) return;
    // line: 12 problem integers, the settings token, then kShareClasses pairs (configuration name, split_k).  A line that
    // does not parse (truncated write, a configuration name this build no longer has) is skipped: its shape is measured again.
    char line[1024];
    while (fgets(line, sizeof(line), f) != nullptr) {
        std::istringstream in(line);
        int v[12];
        bool ok = true;
        for (int i = 0; i < 12 && ok; i++) ok = static_cast<bool>(in >> v[i]);
        std::string token;
        ok = ok && static_cast<bool>(in >> token) && token.find('/') != std::string::npos;
        TunedConv entry;
        for (int c = 0; c < kShareClasses && ok; c++) {
            std::string name;
            int split = 0;
            ok = static_cast<bool>(in >> name >> split) && split >= 1 && split <= 64;
            int variant = -1;
            for (int i = 0; ok && i < conv_num_variants(); i++)
                if (name == conv_variant(i).name) variant = i;
            ok = ok && variant >= 0;
            entry.best[c].variant = variant;
            entry.best[c].split_k = split;
        }
        if (!ok) continue;
        std::ostringstream os;
        for (int i = 0; i < 12; i++) os << (i ? " " : "") << v[i];
        os << ' ' << token;
        // reduced-precision entries have their own keys
        if (conv_variant(entry.best[0].variant).precision == PREC_BF16) os << " bf16";
        if (conv_variant(entry.best[0].variant).precision == PREC_FP16) os << " fp16";
        tuned[os.str()] = entry;
    }
    fclose(f);
}

float *DeviceContext::tuning_buffer(int which, size_t floats) {
    if (floats > tune_floats_[which]) {
        IOS_HIP(hipDeviceSynchronize());
        if (tune_buf_[which] != nullptr) IOS_HIP(hipFree(tune_buf_[which]));
        tune_buf_[which] = nullptr;
        tune_floats_[which] = 0;
        const size_t want = floats + floats / 2 + 1024;
        IOS_HIP(hipMalloc(reinterpret_cast<void **>(&tune_buf_[which]), want * sizeof(float)));
        tune_floats_[which] = want;
        launch_fill_pattern(tune_buf_[which], want, 0x51f15e + which, streams_[0]);
        IOS_HIP(hipStreamSynchronize(streams_[0]));
    }
    return tune_buf_[which];
}

unsigned *DeviceContext::tuning_counters(size_t count) {
    if (count == 0) return nullptr;
    if (count > tune_counter_count_) {
        IOS_HIP(hipDeviceSynchronize());
        if (tune_counters_ != nullptr) IOS_HIP(hipFree(tune_counters_));
        tune_counters_ = nullptr;
        tune_counter_count_ = 0;
        const size_t want = count * 2 + 1024;
        IOS_HIP(hipMalloc(reinterpret_cast<void **>(&tune_counters_), want * sizeof(unsigned)));
        tune_counter_count_ = want;
        launch_fill_u32(tune_counters_, want, 0u, streams_[0]);
        IOS_HIP(hipStreamSynchronize(streams_[0]));
    }
    return tune_counters_;
}

DeviceContext::TunedConv DeviceContext::tune_conv(const ConvProblem &p) {
    // Like the reference's exhaustive algorithm search on first sight of a shape: run every kernel
    // configuration on scratch tensors of the real shape and keep the fastest.
    static const int kSplits[] = {1, 2, 3, 4, 6, 8, 12, 16, 24, 32};
    const size_t kMaxWorkspace = size_t(96) << 20;   // floats
    TensorView x, y;
    x.C = p.IC; x.H = p.H; x.W = p.W; x.bstride = (long long)p.IC * p.H * p.W;
    y.C = p.OC; y.H = p.OH; y.W = p.OW; y.bstride = (long long)p.OC * p.OH * p.OW;
    x.ptr = tuning_buffer(0, (size_t)p.B * x.bstride);
    y.ptr = tuning_buffer(1, (size_t)p.B * y.bstride);
    float *packed = tuning_buffer(2, conv_packed_floats_max(p) + p.OC);
    float *bias = packed + conv_packed_floats_max(p);
    hipStream_t stream = streams_[0];
    struct EventPair {   // destroyed on every way out, a failing launch included
        hipEvent_t start = nullptr, stop = nullptr;
        ~EventPair() {
            if (start != nullptr) (void)hipEventDestroy(start);
            if (stop != nullptr) (void)hipEventDestroy(stop);
        }
    } events;
    IOS_HIP(hipEventCreate(&events.start));
    IOS_HIP(hipEventCreate(&events.stop));
    const hipEvent_t start = events.start, stop = events.stop;
    // one winner per footprint budget: the whole device, a half, a quarter, an eighth (threads in flight);
    // a convolution that shares its stage with other groups uses the winner of the matching budget
    const double capacity = (double)num_cus_ * (double)share_threads_per_cu_;
    struct Candidate {
        ConvLaunch launch;
        float ms;
        double footprint;
        bool fusable;
    };
    auto measure = [&](const ConvLaunch &l, int reps) {
        const size_t ws = conv_workspace_floats(p, l);
        float *workspace = ws ? tuning_buffer(3, ws) : nullptr;
        const SplitKReduce counters = split_reduce(tuning_counters(conv_counter_count(p, l)));
        launch_conv_mfma(p, l, x, packed, bias, y, workspace, counters, stream);   // warm-up
        IOS_HIP(hipEventRecord(start, stream));
        for (int r = 0; r < reps; r++) launch_conv_mfma(p, l, x, packed, bias, y, workspace, counters, stream);
        IOS_HIP(hipEventRecord(stop, stream));
        IOS_HIP(hipEventSynchronize(stop));
        float ms = 0.f;
        IOS_HIP(hipEventElapsedTime(&ms, start, stop));
        return ms / reps;
    };
    // first pass: every configuration and split factor, a few launches each
    std::vector<Candidate> candidates;
    float fastest = 1e30f;
    for (int v = 0; v < conv_num_variants(); v++) {
        const ConvVariant &cv = conv_variant(v);
        if (cv.precision != precision_) continue;   // the precision mode decides which family of configurations competes
        // tiles more than twice as tall / wide as the problem only waste lanes
        if (cv.BM >= 2 * p.OCg() + 32 || cv.BN >= 2 * p.Npix() + 32) continue;
        int last_effective = -1;
        for (int split : kSplits) {
            ConvLaunch l;
            l.variant = v;
            l.split_k = split;
            const int effective = conv_effective_split(p, l);
            if (effective == last_effective) continue;   // asks for more slices than there are K tiles
            last_effective = effective;
            if (conv_workspace_floats(p, l) > kMaxWorkspace) break;
            const float ms = measure(l, 4);
            const double footprint = (double)cv.threads() * ((p.OCg() + cv.BM - 1) / cv.BM) * (double)((p.Npix() + cv.BN - 1) / cv.BN) *
                                     p.groups * effective;
            candidates.push_back({l, ms, footprint, cv.fusable()});
            fastest = std::min(fastest, ms);
            if (ms > 3.f * fastest) break;   // more slices only add reduction work from here on
        }
    }
    // second pass: the three fastest of every class again with more launches (the first pass is noisy at 5-10 us)
    std::sort(candidates.begin(), candidates.end(), [](const Candidate &a, const Candidate &b) { return a.ms < b.ms; });
    std::vector<char> refined(candidates.size(), 0);
    TunedConv result;
    bool found[kShareClasses];
    for (int c = 0; c < kShareClasses; c++) {
        // class 0 is unconstrained; the others accept kernels that fit their share of the device and, under the executors
        // that put the operators of a stage into one launch, can run inside a fused stage launch (the stream and graph
        // executors launch every operator by itself, so every configuration competes); a budget nobody fits takes the
        // fastest such configuration
        const bool any_kernel = !fused_executor();
        // A configuration of the wide-register fused family (three wavefronts per SIMD, items fetched from the table) only
        // competes when it runs for 12 us or more by itself: below that the family's slower start costs more than the
        // kernel gains (Inception-v3 at batch 1, same device: 0.379-0.385 ms with it against 0.375-0.377 ms without).
        constexpr float kWideMinMs = 0.012f;
        auto wide_too_short = [&](const Candidate &cand) {
            return !any_kernel && conv_variant(cand.launch.variant).needs_wide() && cand.ms < kWideMinMs;
        };
        auto eligible = [&](const Candidate &cand, bool fit) {
            if (c == 0) return true;
            if (wide_too_short(cand)) return false;
            return (cand.fusable || any_kernel) && (!fit || cand.footprint <= capacity / (1 << c));
        };
        found[c] = false;
        if (c > 0 && share_cost_rule_) {
            // soft form: time weighted by the share of the device the kernel holds while 2^c - 1 neighbours want theirs
            auto score = [&](const Candidate &cand) { return cand.ms * (1.0 + ((1 << c) - 1) * cand.footprint / capacity); };
            std::vector<size_t> order;
            for (size_t i = 0; i < candidates.size(); i++)
                if ((candidates[i].fusable || any_kernel) && !wide_too_short(candidates[i])) order.push_back(i);
            std::sort(order.begin(), order.end(), [&](size_t a, size_t b) { return score(candidates[a]) < score(candidates[b]); });
            double best = 1e300;
            for (size_t n = 0; n < order.size() && n < 3; n++) {
                Candidate &cand = candidates[order[n]];
                if (!refined[order[n]]) {
                    cand.ms = std::min(cand.ms, measure(cand.launch, 16));
                    refined[order[n]] = 1;
                }
                if (score(cand) < best) {
                    best = score(cand);
                    result.best[c] = cand.launch;
                    found[c] = true;
                }
            }
        }
        for (int pass = 0; pass < 2 && !found[c]; pass++) {
            int taken = 0;
            float best = 1e30f;
            for (size_t i = 0; i < candidates.size() && taken < 3; i++) {
                if (!eligible(candidates[i], pass == 0)) continue;
                taken++;
                if (!refined[i]) {
                    candidates[i].ms = std::min(candidates[i].ms, measure(candidates[i].launch, 16));
                    refined[i] = 1;
                }
                if (candidates[i].ms < best) {
                    best = candidates[i].ms;
                    result.best[c] = candidates[i].launch;
                    found[c] = true;
                }
            }
        }
        if (!found[c]) result.best[c] = conv_pick_launch(p, std::max(1, num_cus_ >> c), c > 0, precision_);
    }
    if (!tune_cache_path_.empty()) {
        FILE *f = fopen(tune_cache_path_.c_str(), "a");
        if (f != nullptr) {
            fprintf(f, "%s %s", conv_signature(p).c_str(), settings_token().c_str());
            for (int c = 0; c < kShareClasses; c++) fprintf(f, " %s %d", conv_variant(result.best[c].variant).name, result.best[c].split_k);
            fprintf(f, "\n");
            fclose(f);
        }
    }
    return result;
}

ConvLaunch DeviceContext::choose_launch(const ConvProblem &p, int share, bool allow_tuning) {
    int cls = 0;
    while (cls + 1 < kShareClasses && (1 << (cls + 1)) <= share) cls++;   // floor(log2(share)), capped
    ConvLaunch launch;
    bool chosen = false;
    if (autotune_) {
        const std::string key = conv_signature(p) + " " + settings_token() + (precision_ == PREC_BF16 ? " bf16" : precision_ == PREC_FP16 ? " fp16" : "");
        auto it = tuned.find(key);
        if (it == tuned.end() && allow_tuning) it = tuned.emplace(key, tune_conv(p)).first;
        if (it != tuned.end()) {
            launch = it->second.best[cls];
            chosen = true;
        }
    }
    if (!chosen) {
        launch = conv_pick_launch(p, std::max(1, num_cus_ >> cls), cls > 0, precision_);
    }
    if (forced_variant_ >= 0) launch.variant = forced_variant_;
    if (forced_split_k_ > 0) launch.split_k = forced_split_k_;
    return launch;
}

float *DeviceContext::shared_arena(size_t floats) {
    if (floats > arena_floats_) {
        IOS_HIP(hipDeviceSynchronize());
        if (arena_ != nullptr) IOS_HIP(hipFree(arena_));
        arena_ = nullptr;
        arena_floats_ = 0;
        const size_t want = floats + floats / 4 + (1u << 20);
        IOS_HIP(hipMalloc(reinterpret_cast<void **>(&arena_), want * sizeof(float)));
        arena_floats_ = want;
        // latency probes run on whatever the arena holds; start from finite, varied values
        launch_fill_pattern(arena_, arena_floats_, 0x1234567u, streams_[0]);
        IOS_HIP(hipStreamSynchronize(streams_[0]));
    }
    return arena_;
}

void *DeviceContext::shared_table(size_t bytes) {
    if (bytes > table_bytes_) {
        IOS_HIP(hipDeviceSynchronize());
        if (table_ != nullptr) IOS_HIP(hipFree(table_));
        table_ = nullptr;
        table_bytes_ = 0;
        const size_t want = bytes * 2 + 4096;
        IOS_HIP(hipMalloc(&table_, want));
        table_bytes_ = want;
    }
    return table_;
}

void DeviceContext::set_option(const std::string &key, const std::string &value) {
    if (key == "executor") {
        if (value == "streams") exec_mode_ = ExecMode::Streams;
        else if (value == "graph") exec_mode_ = ExecMode::Graph;
        else if (value == "fused") exec_mode_ = ExecMode::Fused;
        else if (value == "fused_graph") exec_mode_ = ExecMode::FusedGraph;
        else throw std::runtime_error("option executor: expected streams, graph, fused or fused_graph, got '" + value + "'");
    } else if (key == "autotune") {
        autotune_ = !(value == "0" || value == "false" || value == "off" || value.empty());
    } else if (key == "conv_variant") {
        const int v = atoi(value.c_str());
        if (v < -1 || v >= conv_num_variants()) throw std::runtime_error("option conv_variant: index out of range");
        forced_variant_ = v;
    } else if (key == "conv_split_k") {
        const int v = atoi(value.c_str());
        if (v < 0 || v > 64) throw std::runtime_error("option conv_split_k: expected 0..64");
        forced_split_k_ = v;
    } else if (key == "share_rule") {
        if (value == "cost") share_cost_rule_ = true;
        else if (value == "budget") share_cost_rule_ = false;
        else throw std::runtime_error("option share_rule: expected cost or budget");
    } else if (key == "share_threads_per_cu") {
        const int v = atoi(value.c_str());
        if (v < 64 || v > 4096) throw std::runtime_error("option share_threads_per_cu: expected 64..4096");
        share_threads_per_cu_ = v;
    } else if (key == "precision") {
        if (value == "fp32") precision_ = PREC_FP32;
        else if (value == "bf16") precision_ = PREC_BF16;
        else if (value == "fp16") precision_ = PREC_FP16;
        else throw std::runtime_error("option precision: expected fp32, bf16 or fp16, got '" + value + "'");
    } else if (key == "split_k_reduce") {
        if (value == "xcd") reduce_mode_ = ReduceMode::Xcd;   // (falls back to inline where the placement probe failed)
        else if (value == "inline") reduce_mode_ = ReduceMode::Inline;
        else if (value == "kernel") reduce_mode_ = ReduceMode::Kernel;
        else throw std::runtime_error("option split_k_reduce: expected xcd, inline or kernel, got '" + value + "'");
    } else if (key == "clear_tuning") {
        tuned.clear();
    } else {
        throw std::runtime_error("unknown option '" + key + "'");
    }
}

std::string DeviceContext::info_json() const {
    std::ostringstream os;
    os << "{\"name\":\"" << name_ << "\",\"arch\":\"" << arch_ << "\",\"compute_units\":" << num_cus_
       << ",\"executor\":\"" << (exec_mode_ == ExecMode::Graph ? "graph" : exec_mode_ == ExecMode::Fused ? "fused" : exec_mode_ == ExecMode::FusedGraph ? "fused_graph" : "streams") << "\",\"autotune\":" << (autotune_ ? "true" : "false")
       << ",\"split_k_reduce\":\"" << (reduce_mode_ == ReduceMode::Xcd ? "xcd" : reduce_mode_ == ReduceMode::Inline ? "inline" : "kernel") << "\""
       << ",\"xcd_placement_probe\":" << (xcd_usable_ ? "true" : "false") << ",\"xcd_map\":" << xcd_map_[0]
       << ",\"precision\":\"" << (precision_ == PREC_BF16 ? "bf16" : precision_ == PREC_FP16 ? "fp16" : "fp32") << "\""
       << ",\"conv_variant\":" << forced_variant_ << ",\"conv_split_k\":" << forced_split_k_
       << ",\"arena_reuse\":" << (planner_arena_reuse() ? "true" : "false")
       << ",\"max_groups\":" << kMaxGroups << ",\"conv_variants\":[";
    for (int i = 0; i < conv_num_variants(); i++) os << (i ? "," : "") << '"' << conv_variant(i).name << '"';
    os << "]}";
    return os.str();
}

// ---- session ---------------------------------------------------------------------------------------------------------
Session::Session(Plan plan, Storage storage) : plan_(std::move(plan)), ctx_(DeviceContext::get()) {
    if (storage == Storage::Static) {
        const size_t need = plan_.arena_floats * sizeof(float);
        if (need > DeviceContext::static_scratch_bytes())
            throw std::runtime_error("graph needs " + std::to_string(need) + " bytes of device memory at this batch size; the static scratch of "
                                     "graph_inference_no_alloc holds " + std::to_string(DeviceContext::static_scratch_bytes()));
        base_ = ctx_.static_scratch();
        owns_memory_ = false;
        static_ = true;
    } else if (storage == Storage::Shared) {
        base_ = ctx_.shared_arena(plan_.arena_floats);
        owns_memory_ = false;
    } else {
        IOS_HIP(hipMalloc(reinterpret_cast<void **>(&base_), std::max<size_t>(plan_.arena_floats, 64) * sizeof(float)));
        owns_memory_ = true;
    }
    try {
        setup();
    } catch (...) {
        release();   // the destructor does not run for a constructor that throws
        throw;
    }
}

Session::~Session() { release(); }

void Session::release() noexcept {
    (void)hipDeviceSynchronize();
    if (graph_exec_ != nullptr) (void)hipGraphExecDestroy(graph_exec_);
    if (graph_ != nullptr) (void)hipGraphDestroy(graph_);
    for (hipEvent_t e : fork_events_)
        if (e != nullptr) (void)hipEventDestroy(e);
    for (auto &per_stage : join_events_)
        for (hipEvent_t e : per_stage) (void)hipEventDestroy(e);
    for (hipEvent_t e : stage_events_) (void)hipEventDestroy(e);
    if (start_ != nullptr) (void)hipEventDestroy(start_);
    if (stop_ != nullptr) (void)hipEventDestroy(stop_);
    if (owns_memory_ && fused_items_ != nullptr) (void)hipFree(fused_items_);
    if (owns_memory_ && base_ != nullptr) (void)hipFree(base_);
    graph_exec_ = nullptr;
    graph_ = nullptr;
    fork_events_.clear();
    join_events_.clear();
    stage_events_.clear();
    start_ = stop_ = nullptr;
    fused_items_ = nullptr;
    base_ = nullptr;
}

TensorView Session::tv(const ViewRef &v) const {
    TensorView t;
    t.ptr = base_ + v.offset;
    t.C = v.C;
    t.H = v.H;
    t.W = v.W;
    t.bstride = v.bstride;
    return t;
}

void Session::setup() {
    hipStream_t main = ctx_.stream(0);
    if (owns_memory_) launch_fill_pattern(base_, plan_.arena_floats, 0x2468aceu, main);
    for (const PlanConv &conv : plan_.convs) {
        // a convolution in front of the average pool it was exchanged with adds zeros; the pool adds the bias
        if (conv.linear) launch_fill_u32(reinterpret_cast<unsigned *>(base_ + conv.zero_bias_off), (size_t)conv.problem.OC, 0u, main);
        if (!conv.matrix_path) continue;
        // the probes never upload filters: pack whatever the filter region holds so that the matrix
        // path reads initialised memory
        launch_pack_filters(conv.problem, conv.launch, base_ + conv.weight_off, base_ + conv.packed_off, main);
        // split-K tickets start at zero; every launch leaves them at zero again
        if (conv.ctr_count > 0) launch_fill_u32(reinterpret_cast<unsigned *>(base_ + conv.ctr_off), conv.ctr_count, 0u, main);
    }
    const size_t num_stages = plan_.stages.size();
    if (static_) {   // no events: everything is issued on the main stream and the host waits for the stream
        IOS_HIP(hipStreamSynchronize(main));
        return;
    }
    fork_events_.assign(num_stages, nullptr);
    join_events_.assign(num_stages, {});
    for (size_t s = 0; s < num_stages; s++) {
        const size_t groups = plan_.stages[s].size();
        if (groups <= 1) continue;
        IOS_HIP(hipEventCreateWithFlags(&fork_events_[s], hipEventDisableTiming));
        join_events_[s].resize(groups - 1);
        for (hipEvent_t &e : join_events_[s]) IOS_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
    }
    IOS_HIP(hipEventCreate(&start_));
    IOS_HIP(hipEventCreate(&stop_));
    IOS_HIP(hipStreamSynchronize(main));
}

void Session::set_input(const float *host) {
    if (host == nullptr) throw std::runtime_error("input pointer is null");
    hipStream_t main = ctx_.stream(0);
    const ViewRef &in = plan_.input;
    IOS_HIP(hipMemcpyAsync(base_ + in.offset, host, (size_t)plan_.batch * in.image_floats() * sizeof(float), hipMemcpyHostToDevice, main));
    IOS_HIP(hipStreamSynchronize(main));
}

bool Session::set_conv_weights(const char *name, const float *weight, const float *bias) {
    auto it = plan_.conv_index.find(name ? name : "");
    if (it == plan_.conv_index.end()) {
        printf("%s not found\n", name ? name : "(null)");
        return false;
    }
    if (weight == nullptr || bias == nullptr) throw std::runtime_error(std::string("convolution '") + name + "': weight or bias pointer is null");
    const PlanConv &conv = plan_.convs[it->second];
    const ConvProblem &p = conv.problem;
    hipStream_t main = ctx_.stream(0);
    IOS_HIP(hipMemcpyAsync(base_ + conv.weight_off, weight, (size_t)p.OC * p.K() * sizeof(float), hipMemcpyHostToDevice, main));
    IOS_HIP(hipMemcpyAsync(base_ + conv.bias_off, bias, (size_t)p.OC * sizeof(float), hipMemcpyHostToDevice, main));
    if (conv.matrix_path) launch_pack_filters(p, conv.launch, base_ + conv.weight_off, base_ + conv.packed_off, main);
    IOS_HIP(hipStreamSynchronize(main));
    return true;
}

void Session::copy_out(const ViewRef &view, float *host) {
    hipStream_t main = ctx_.stream(0);
    const size_t image = view.image_floats();
    if (view.bstride == (long long)image) {
        IOS_HIP(hipMemcpyAsync(host, base_ + view.offset, (size_t)plan_.batch * image * sizeof(float), hipMemcpyDeviceToHost, main));
    } else {
        for (int b = 0; b < plan_.batch; b++)
            IOS_HIP(hipMemcpyAsync(host + (size_t)b * image, base_ + view.offset + (size_t)b * view.bstride, image * sizeof(float),
                                   hipMemcpyDeviceToHost, main));
    }
    IOS_HIP(hipStreamSynchronize(main));
}

void Session::get_output(float *host) {
    if (host == nullptr) throw std::runtime_error("output pointer is null");
    if (!plan_.output_single_group) throw std::runtime_error("the last stage of the schedule must have a single group");
    copy_out(plan_.output, host);
}

void Session::get_tensor(const std::string &name, float *host) {
    auto it = plan_.tensors.find(name);
    if (it == plan_.tensors.end()) throw std::runtime_error("operator '" + name + "' has no materialised output");
    if (plan_.overwritten.count(name))
        throw std::runtime_error("the output of operator '" + name + "' shares its memory with a later operator and does not survive the pass "
                                 "(option arena_reuse=0 keeps every output)");
    copy_out(it->second, host);
}

unsigned *Session::counters_of(const PlanConv &c) const {
    if (c.ctr_count == 0 || !ctx_.inline_reduce()) return nullptr;
    return reinterpret_cast<unsigned *>(base_ + c.ctr_off);
}

void Session::launch_op(const PlanOp &op, int group) {
    hipStream_t stream = ctx_.stream(group);
    switch (op.kind) {
        case OpKind::ConvMfma: {
            const PlanConv &c = plan_.convs[op.conv];
            const TensorView residual = op.has_residual ? tv(op.residual) : TensorView{};
            launch_conv_mfma(c.problem, c.launch, tv(op.in), base_ + c.packed_off, bias_of(c), tv(op.out),
                             c.ws_floats ? base_ + c.ws_off : nullptr, ctx_.split_reduce(counters_of(c), group, !capturing_forks_), stream,
                             op.has_residual ? &residual : nullptr,
                             op.post_relu != 0);
            break;
        }
        case OpKind::ConvDepthwise: {
            const PlanConv &c = plan_.convs[op.conv];
            TensorView more[kMaxNaryInputs];
            for (size_t i = 1; i < op.srcs.size(); i++) more[i - 1] = tv(op.srcs[i]);
            launch_dwconv(c.problem, tv(op.in), base_ + c.weight_off, bias_of(c), tv(op.out), stream, more,
                          op.srcs.empty() ? 0 : (int)op.srcs.size() - 1);
            break;
        }
        case OpKind::ConvDirect: {
            const PlanConv &c = plan_.convs[op.conv];
            launch_conv_direct(c.problem, tv(op.in), base_ + c.weight_off, bias_of(c), tv(op.out), stream, c.thin);
            break;
        }
        case OpKind::Pool:
            launch_pool(op.pool, tv(op.in), tv(op.out), stream, op.bias_conv >= 0 ? base_ + plan_.convs[op.bias_conv].bias_off : nullptr, op.act);
            break;
        case OpKind::GlobalPool: launch_global_pool(op.pool, tv(op.in), tv(op.out), stream); break;
        case OpKind::Nary: {
            NaryArgs a;
            a.count = (int)op.srcs.size();
            for (int i = 0; i < a.count; i++) {
                a.src[i] = base_ + op.srcs[i].offset;
                a.src_bstride[i] = op.srcs[i].bstride;
            }
            launch_nary(a, op.multiply, op.accumulate, op.act, plan_.batch, (long long)op.out.image_floats(), tv(op.out), stream);
            break;
        }
        case OpKind::Unary: launch_unary(tv(op.in), tv(op.out), op.act, plan_.batch, stream); break;
    }
}

void Session::enqueue_streams(bool stage_events) {
    hipStream_t main = ctx_.stream(0);
    for (size_t s = 0; s < plan_.stages.size(); s++) {
        const auto &groups = plan_.stages[s];
        const bool fork = groups.size() > 1;
        if (fork) {
            IOS_HIP(hipEventRecord(fork_events_[s], main));
            for (size_t g = 1; g < groups.size(); g++) IOS_HIP(hipStreamWaitEvent(ctx_.stream((int)g), fork_events_[s], 0));
        }
        for (size_t g = 0; g < groups.size(); g++)
            for (int op : groups[g]) launch_op(plan_.ops[op], (int)g);
        if (fork) {
            for (size_t g = 1; g < groups.size(); g++) {
                IOS_HIP(hipEventRecord(join_events_[s][g - 1], ctx_.stream((int)g)));
                IOS_HIP(hipStreamWaitEvent(main, join_events_[s][g - 1], 0));
            }
        }
        if (stage_events) IOS_HIP(hipEventRecord(stage_events_[s], main));
    }
}

void Session::enqueue_serial() {
    hipStream_t main = ctx_.stream(0);
    for (const auto &groups : plan_.stages)
        for (const auto &group : groups)
            for (int op : group) launch_op(plan_.ops[op], 0);
}

void Session::enqueue(bool stage_events) {
    if (static_) {
        if (stage_events) throw std::runtime_error("a session in the static scratch cannot profile stages");
        enqueue_serial();
        return;
    }
    const ExecMode mode = ctx_.exec_mode();
    if (mode == ExecMode::Fused || mode == ExecMode::FusedGraph) enqueue_fused(stage_events);
    else enqueue_streams(stage_events);
}

// ---- fused stage launches -----------------------------------------------------------------------------------------
// A stage is cut into levels: the operations of a group follow each other, except that operations of one unit on the same
// PlanOp::level (the terms of a concatenation) share a level; a split-K convolution contributes its main kernel and, with
// the two-kernel reduction, one level later its reduction.  The kernels of one level are independent and become work items
// of one fused launch; levels follow each other on the main stream.  A single-group stage keeps its stand-alone kernels on
// the levels that hold one operation.
void Session::build_fused() {
    if (fused_built_) return;
    std::vector<WorkItem> items;
    fused_stages_.assign(plan_.stages.size(), {});
    struct Pending {
        WorkItem item;
        int threads;     // 0: any block size
        int smem_bytes;
        int op;          // plan operation behind the item
        bool fusable;
    };
    for (size_t s = 0; s < plan_.stages.size(); s++) {
        const auto &groups = plan_.stages[s];
        const bool solo = groups.size() <= 1;
        if (solo) {
            bool shared_level = false;
            for (const auto &group : groups)
                for (size_t i = 1; i < group.size(); i++) {
                    const PlanOp &a = plan_.ops[group[i - 1]], &b = plan_.ops[group[i]];
                    if (a.unit == b.unit && a.level == b.level) shared_level = true;
                }
            if (!shared_level) continue;
        }
        std::vector<std::vector<std::vector<Pending>>> chains(groups.size());   // group, level, items
        for (size_t g = 0; g < groups.size(); g++) {
            auto &chain = chains[g];
            int unit = -2;
            size_t base = 0, shift = 0;
            auto level_of = [&](const PlanOp &op) -> std::vector<Pending> & {
                if (op.unit != unit) {
                    unit = op.unit;
                    base = chain.size();
                    shift = 0;
                }
                const size_t at = base + shift + (size_t)op.level;
                if (chain.size() <= at) chain.resize(at + 1);
                return chain[at];
            };
            for (int index : groups[g]) {
                const PlanOp &op = plan_.ops[index];
                Pending pend;
                memset(&pend.item, 0, sizeof(WorkItem));
                pend.threads = 0;
                pend.smem_bytes = 0;
                pend.op = index;
                pend.fusable = true;
                int blocks = 0;
                switch (op.kind) {
                    case OpKind::ConvMfma: {
                        const PlanConv &c = plan_.convs[op.conv];
                        const TensorView residual = op.has_residual ? tv(op.residual) : TensorView{};
                        const ConvDispatch d = make_conv_dispatch(c.problem, c.launch, tv(op.in), base_ + c.packed_off, bias_of(c),
                                                                  tv(op.out), c.ws_floats ? base_ + c.ws_off : nullptr, ctx_.split_reduce(counters_of(c)),
                                                                  op.has_residual ? &residual : nullptr, op.post_relu != 0);
                        pend.fusable = conv_variant(d.variant).fusable() && !op.has_residual;   // (the fused kernel holds the plain epilogue)
                        if (!pend.fusable && !solo)
                            throw std::runtime_error(op.has_residual ? std::string("internal: a residual convolution is planned for single-group stages only")
                                                                     : std::string("convolution kernel configuration ") + conv_variant(d.variant).name +
                                                                           " cannot run inside a fused stage launch");
                        pend.item.kind = WORK_CONV;
                        pend.item.variant = d.variant;
                        pend.item.tiles = d.tiles;
                        pend.item.groups = d.groups;
                        pend.item.div_tiles = make_fast_div((unsigned)d.tiles);
                        pend.item.div_groups = make_fast_div((unsigned)d.groups);
                        pend.item.num_blocks = d.grid_blocks();
                        pend.item.conv = d.args;
                        pend.threads = d.threads;
                        pend.smem_bytes = d.smem_bytes;
                        if (d.has_reduce && solo) pend.fusable = false;   // launched stand-alone, reduction included
                        level_of(op).push_back(pend);
                        if (d.has_reduce && !solo) {
                            Pending red;
                            memset(&red.item, 0, sizeof(WorkItem));
                            red.item.kind = WORK_REDUCE;
                            red.item.num_blocks = d.reduce_blocks;
                            red.item.reduce = d.reduce;
                            red.threads = 0;
                            red.smem_bytes = 0;
                            red.op = index;
                            red.fusable = true;
                            shift++;
                            level_of(op).push_back(red);
                        }
                        continue;
                    }
                    case OpKind::ConvDepthwise:
                    case OpKind::ConvDirect: {
                        const PlanConv &c = plan_.convs[op.conv];
                        pend.item.kind = op.kind == OpKind::ConvDepthwise ? WORK_DWCONV : WORK_CONV_DIRECT;
                        if (c.thin) throw std::runtime_error("internal: the thin-input convolution kernel is planned for single-group stages only");
                        pend.item.direct = make_direct_conv_args(c.problem, tv(op.in), base_ + c.weight_off, bias_of(c), tv(op.out), &blocks);
                        if (op.kind == OpKind::ConvDepthwise && op.srcs.size() > 1) {
                            TensorView more[kMaxNaryInputs];
                            for (size_t i = 1; i < op.srcs.size(); i++) more[i - 1] = tv(op.srcs[i]);
                            add_dwconv_sources(pend.item.direct, more, (int)op.srcs.size() - 1);
                        }
                        break;
                    }
                    case OpKind::Pool:
                    case OpKind::GlobalPool:
                        pend.item.kind = op.kind == OpKind::Pool ? WORK_POOL : WORK_GLOBAL_POOL;
                        pend.item.pool = make_pool_args(op.pool, tv(op.in), tv(op.out), op.kind == OpKind::GlobalPool, &blocks,
                                                        op.bias_conv >= 0 ? base_ + plan_.convs[op.bias_conv].bias_off : nullptr, op.act);
                        break;
                    case OpKind::Nary:
                    case OpKind::Unary: {
                        NaryArgs in;
                        if (op.kind == OpKind::Unary) {
                            in.count = 1;
                            in.src[0] = base_ + op.in.offset;
                            in.src_bstride[0] = op.in.bstride;
                        } else {
                            in.count = (int)op.srcs.size();
                            for (int i = 0; i < in.count; i++) {
                                in.src[i] = base_ + op.srcs[i].offset;
                                in.src_bstride[i] = op.srcs[i].bstride;
                            }
                        }
                        pend.item.kind = WORK_NARY;
                        pend.item.nary = make_nary_args(in, op.multiply, op.accumulate, op.act, plan_.batch,
                                                        (long long)op.out.image_floats(), tv(op.out), &blocks);
                        break;
                    }
                }
                pend.item.num_blocks = blocks;   // sized for 256-thread blocks, rescaled below
                level_of(op).push_back(pend);
            }
        }
        size_t depth = 0;
        for (const auto &chain : chains) depth = std::max(depth, chain.size());
        for (size_t level = 0; level < depth; level++) {
            std::vector<Pending *> here;
            int widest = 0;
            bool all_fusable = true;
            for (auto &chain : chains)
                if (level < chain.size())
                    for (Pending &pend : chain[level]) {
                        here.push_back(&pend);
                        widest = std::max(widest, pend.threads);
                        all_fusable = all_fusable && pend.fusable;
                    }
            if (here.empty()) continue;
            // a configuration of the wide-register family beside a 1024-thread body: that family has no such form, the
            // operators of the level are launched one after the other instead (they are independent of each other)
            bool needs_wide = false;
            for (Pending *pend : here)
                needs_wide = needs_wide || (pend->item.kind == WORK_CONV && conv_variant(pend->item.variant).needs_wide());
            if (needs_wide && widest > 512 && all_fusable) {
                for (Pending *pend : here)
                    if (pend->item.kind != WORK_REDUCE)   // (a stand-alone split-K launch brings its own reduction)
                        fused_stages_[s].push_back(FusedLaunch{0, 0, 0, 0, 0, pend->op, {}, {pend->op}});
                continue;
            }
            if (solo && (here.size() == 1 || !all_fusable)) {
                for (Pending *pend : here) fused_stages_[s].push_back(FusedLaunch{0, 0, 0, 0, 0, pend->op, {}, {pend->op}});
                continue;
            }
            widest = std::max(widest, 256);   // narrowest instantiation of the fused kernel
            // one launch per level, as wide as its widest convolution body; more items than a launch holds: several launches
            for (size_t first = 0; first < here.size(); first += kMaxFusedItems) {
                const size_t last = std::min(here.size(), first + (size_t)kMaxFusedItems);
                FusedLaunch launch{widest, (int)items.size(), 0, 0, 0, -1, {}, {}};
                for (size_t i = first; i < last; i++) {
                    Pending *pend = here[i];
                    launch.ops.push_back(pend->op);
                    WorkItem item = pend->item;
                    item.threads = pend->threads == 0 ? widest : pend->threads;
                    if (pend->threads == 0) item.num_blocks = std::max(1, (item.num_blocks * 256 + widest - 1) / widest);
                    item.first_block = launch.total_blocks;
                    if (launch.num_items < kFusedHeaderItems) launch.header.first_block[launch.num_items] = item.first_block;
                    launch.total_blocks += item.num_blocks;
                    launch.smem_bytes = std::max(launch.smem_bytes, pend->smem_bytes);
                    launch.num_items++;
                    items.push_back(item);
                }
                launch.header.num_items = launch.num_items;
                fused_stages_[s].push_back(launch);
            }
        }
    }
    fused_items_host_ = items;
    if (!items.empty()) {
        if (owns_memory_) IOS_HIP(hipMalloc(&fused_items_, items.size() * sizeof(WorkItem)));
        else fused_items_ = ctx_.shared_table(items.size() * sizeof(WorkItem));
        IOS_HIP(hipMemcpyAsync(fused_items_, items.data(), items.size() * sizeof(WorkItem), hipMemcpyHostToDevice, ctx_.stream(0)));
        IOS_HIP(hipStreamSynchronize(ctx_.stream(0)));
    }
    fused_built_ = true;
}

void Session::enqueue_fused(bool stage_events) {
    build_fused();
    hipStream_t main = ctx_.stream(0);
    const WorkItem *items = static_cast<const WorkItem *>(fused_items_);
    for (size_t s = 0; s < plan_.stages.size(); s++) {
        if (fused_stages_[s].empty()) {
            for (const auto &group : plan_.stages[s])
                for (int op : group) launch_op(plan_.ops[op], 0);
        } else {
            for (const FusedLaunch &l : fused_stages_[s]) {
                if (l.single_op >= 0) launch_op(plan_.ops[l.single_op], 0);
                else launch_fused(l.threads, items + l.first_item, fused_items_host_.data() + l.first_item, l.header, l.total_blocks, l.smem_bytes, ctx_.num_cus(), main);
            }
        }
        if (stage_events) IOS_HIP(hipEventRecord(stage_events_[s], main));
    }
}

void Session::build_graph() {
    hipStream_t main = ctx_.stream(0);
    IOS_HIP(hipStreamBeginCapture(main, hipStreamCaptureModeRelaxed));
    // the stream executor forks inside the capture, and the replay runs the branches on streams of its own choice
    capturing_forks_ = ctx_.exec_mode() == ExecMode::Graph;
    try {
        enqueue(false);
        capturing_forks_ = false;
    } catch (...) {
        capturing_forks_ = false;
        hipGraph_t broken = nullptr;
        (void)hipStreamEndCapture(main, &broken);
        if (broken != nullptr) (void)hipGraphDestroy(broken);
        throw;
    }
    IOS_HIP(hipStreamEndCapture(main, &graph_));
    IOS_HIP(hipGraphInstantiate(&graph_exec_, graph_, nullptr, nullptr, 0));
}

void Session::forward() {
    if (static_) {
        enqueue_serial();
        return;
    }
    const ExecMode mode = ctx_.exec_mode();
    if (mode == ExecMode::Graph || mode == ExecMode::FusedGraph) {
        if (graph_exec_ != nullptr && graph_mode_ != mode) {   // the option changed since the capture
            IOS_HIP(hipGraphExecDestroy(graph_exec_));
            IOS_HIP(hipGraphDestroy(graph_));
            graph_exec_ = nullptr;
            graph_ = nullptr;
        }
        if (graph_exec_ == nullptr) {
            if (mode == ExecMode::FusedGraph) build_fused();   // allocations and copies stay outside the capture
            build_graph();
            graph_mode_ = mode;
        }
        IOS_HIP(hipGraphLaunch(graph_exec_, ctx_.stream(0)));
    } else {
        enqueue(false);
    }
}

void Session::run() {
    forward();
    synchronize();
}

void Session::synchronize() {
    IOS_HIP(hipStreamSynchronize(ctx_.stream(0)));
    ctx_.check_xcd_fault();
}

void Session::measure(int warmup, int number, int repeat, bool profile_stage, float *results, float *stage_results) {
    if (static_) throw std::runtime_error("a session in the static scratch has no timers");
    if (number < 1 || repeat < 1 || warmup < 0) throw std::runtime_error("measure: warmup >= 0, number >= 1, repeat >= 1 required");
    hipStream_t main = ctx_.stream(0);
    const size_t num_stages = plan_.stages.size();
    if (profile_stage && stage_events_.empty()) {
        stage_events_.resize(num_stages);
        for (hipEvent_t &e : stage_events_) IOS_HIP(hipEventCreate(&e));
    }
    auto pass = [&]() {
        if (profile_stage) enqueue(true);
        else forward();
    };
    for (int i = 0; i < warmup; i++) pass();
    for (int i = 0; i < repeat; i++) {
        double total = 0.0;
        std::vector<double> per_stage(num_stages, 0.0);
        for (int t = 0; t < number; t++) {
            IOS_HIP(hipDeviceSynchronize());
            IOS_HIP(hipEventRecord(start_, main));
            pass();
            IOS_HIP(hipEventRecord(stop_, main));
            IOS_HIP(hipEventSynchronize(stop_));
            float ms = 0.f;
            if (profile_stage) {
                for (size_t s = 0; s < num_stages; s++) {
                    hipEvent_t from = s == 0 ? start_ : stage_events_[s - 1];
                    hipEvent_t to = s + 1 == num_stages ? stop_ : stage_events_[s];
                    IOS_HIP(hipEventElapsedTime(&ms, from, to));
                    per_stage[s] += ms;
                }
            }
            IOS_HIP(hipEventElapsedTime(&ms, start_, stop_));
            total += ms;
        }
        results[i] = (float)(total / number);
        if (profile_stage && stage_results != nullptr)
            for (size_t s = 0; s < num_stages; s++) stage_results[i * num_stages + s] = (float)(per_stage[s] / number);
    }
    IOS_HIP(hipDeviceSynchronize());
    ctx_.check_xcd_fault();
}

void Session::measure_back_to_back(int warmup, int number, int repeat, float *results) {
    if (static_) throw std::runtime_error("a session in the static scratch has no timers");
    if (number < 1 || repeat < 1 || warmup < 0) throw std::runtime_error("measure: warmup >= 0, number >= 1, repeat >= 1 required");
    hipStream_t main = ctx_.stream(0);
    for (int i = 0; i < warmup; i++) forward();
    for (int i = 0; i < repeat; i++) {
        IOS_HIP(hipDeviceSynchronize());
        IOS_HIP(hipEventRecord(start_, main));
        for (int t = 0; t < number; t++) forward();
        IOS_HIP(hipEventRecord(stop_, main));
        IOS_HIP(hipEventSynchronize(stop_));
        float ms = 0.f;
        IOS_HIP(hipEventElapsedTime(&ms, start_, stop_));
        results[i] = ms / (float)number;
    }
    IOS_HIP(hipDeviceSynchronize());
    ctx_.check_xcd_fault();
}

void Session::profile_ops(int warmup, int repeat, float *ms_out) {
    if (static_) throw std::runtime_error("a session in the static scratch has no timers");
    if (repeat < 1 || warmup < 0) throw std::runtime_error("profile_ops: warmup >= 0 and repeat >= 1 required");
    hipStream_t main = ctx_.stream(0);
    run();   // every operator sees the inputs it has in a real pass
    for (size_t i = 0; i < plan_.ops.size(); i++) {
        const PlanOp &op = plan_.ops[i];
        for (int w = 0; w < warmup; w++) launch_op(op, 0);
        IOS_HIP(hipStreamSynchronize(main));
        IOS_HIP(hipEventRecord(start_, main));
        for (int r = 0; r < repeat; r++) launch_op(op, 0);
        IOS_HIP(hipEventRecord(stop_, main));
        IOS_HIP(hipEventSynchronize(stop_));
        float ms = 0.f;
        IOS_HIP(hipEventElapsedTime(&ms, start_, stop_));
        ms_out[i] = ms / (float)repeat;
    }
}

// ---- per-launch view of a pass -------------------------------------------------------------------------------------------
static std::string op_kernel_name(const Plan &plan, const PlanOp &op) {
    switch (op.kind) {
        case OpKind::ConvMfma: return std::string("conv_kernel<") + conv_variant(plan.convs[op.conv].launch.variant).name + ">";
        case OpKind::ConvDepthwise: return "dwconv_kernel";
        case OpKind::ConvDirect: return plan.convs[op.conv].thin ? "conv_thin_kernel" : "conv_direct_kernel";
        case OpKind::Pool: return "pool_kernel";
        case OpKind::GlobalPool: return "global_pool_kernel";
        case OpKind::Nary:
        case OpKind::Unary: return "nary_kernel";
    }
    return "?";
}

std::vector<Session::LaunchRecord> Session::launches() {
    const ExecMode mode = ctx_.exec_mode();
    const bool fused = !static_ && (mode == ExecMode::Fused || mode == ExecMode::FusedGraph);
    if (fused) build_fused();
    std::vector<LaunchRecord> out;
    for (size_t s = 0; s < plan_.stages.size(); s++) {
        const auto &groups = plan_.stages[s];
        if (fused && !fused_stages_[s].empty()) {
            for (size_t l = 0; l < fused_stages_[s].size(); l++) {
                const FusedLaunch &f = fused_stages_[s][l];
                LaunchRecord r;
                r.stage = (int)s;
                if (f.single_op >= 0) {
                    r.kernel = op_kernel_name(plan_, plan_.ops[f.single_op]);
                    r.ops = {f.single_op};
                    out.push_back(r);
                    continue;
                }
                const FusedForm form = fused_launch_form(fused_items_host_.data() + f.first_item, f.num_items, f.threads, f.total_blocks, ctx_.num_cus());
                r.kernel = std::string(fused_kernel_name(form)) + "<" + std::to_string(f.threads) + ">";
                r.ops = f.ops;
                r.blocks = f.total_blocks;
                r.threads = f.threads;
                r.fused_level = (int)l;
                out.push_back(r);
            }
            continue;
        }
        for (const auto &group : groups)
            for (int index : group) {
                LaunchRecord r;
                r.stage = (int)s;
                r.kernel = op_kernel_name(plan_, plan_.ops[index]);
                r.ops = {index};
                out.push_back(r);
            }
    }
    return out;
}

std::string Session::describe_launches() {
    std::ostringstream os;
    os << '[';
    bool first = true;
    for (const LaunchRecord &r : launches()) {
        double flops = 0.0, bytes = 0.0, conv_flops = 0.0;
        std::vector<int> seen;
        for (int index : r.ops) {
            if (std::find(seen.begin(), seen.end(), index) != seen.end()) continue;
            seen.push_back(index);
            flops += plan_.ops[index].flops;
            bytes += plan_.ops[index].bytes;
            if (plan_.ops[index].kind == OpKind::ConvMfma) conv_flops += plan_.ops[index].flops;
        }
        os << (first ? "" : ",") << "{\"stage\":" << r.stage << ",\"kernel\":\"" << r.kernel << "\",\"fused_level\":" << r.fused_level
           << ",\"blocks\":" << r.blocks << ",\"threads\":" << r.threads << ",\"flops\":" << flops << ",\"matrix_flops\":" << conv_flops
           << ",\"bytes\":" << bytes << ",\"ops\":[";
        for (size_t i = 0; i < seen.size(); i++) os << (i ? "," : "") << seen[i];
        os << "]}";
        first = false;
    }
    os << ']';
    return os.str();
}

void Session::profile_launches(int warmup, int repeat, float *ms_out, int capacity) {
    if (static_) throw std::runtime_error("a session in the static scratch has no timers");
    if (repeat < 1 || warmup < 0) throw std::runtime_error("profile_launches: warmup >= 0 and repeat >= 1 required");
    const std::vector<LaunchRecord> list = launches();
    if ((int)list.size() > capacity) throw std::runtime_error("profile_launches: output array too small");
    hipStream_t main = ctx_.stream(0);
    run();   // every launch sees the inputs it has in a real pass
    const WorkItem *items = static_cast<const WorkItem *>(fused_items_);
    for (size_t i = 0; i < list.size(); i++) {
        const LaunchRecord &r = list[i];
        auto issue = [&]() {
            if (r.fused_level >= 0) {
                const FusedLaunch &l = fused_stages_[r.stage][r.fused_level];
                launch_fused(l.threads, items + l.first_item, fused_items_host_.data() + l.first_item, l.header, l.total_blocks, l.smem_bytes, ctx_.num_cus(), main);
            } else {
                launch_op(plan_.ops[r.ops[0]], 0);
            }
        };
        for (int w = 0; w < warmup; w++) issue();
        IOS_HIP(hipStreamSynchronize(main));
        IOS_HIP(hipEventRecord(start_, main));
        for (int k = 0; k < repeat; k++) issue();
        IOS_HIP(hipEventRecord(stop_, main));
        IOS_HIP(hipEventSynchronize(stop_));
        float ms = 0.f;
        IOS_HIP(hipEventElapsedTime(&ms, start_, stop_));
        ms_out[i] = ms / (float)repeat;
    }
}

}  // namespace ios
