// C ABI of libios_runtime.so.  Declarations and the reference interfaces they stand in for are in
// include/ios_runtime.h.  Every entry point catches C++ exceptions, stores the message for
// ios_last_error() and returns a non-zero status instead of terminating the host process.
#include <cstdio>
#include <cstring>
#include <memory>
#include <mutex>
#include <string>

#include "../../include/ios_runtime.h"
#include "plan.h"
#include "runtime.h"
#include "conv_body.h"

namespace {

std::string g_last_error;
// The library keeps process-wide state (device context, stream pool, shared arena, configuration cache); calls from
// several host threads are serialised here rather than left to race.
std::recursive_mutex g_api_mutex;

ios::LaunchChooser device_chooser() {
    ios::DeviceContext &ctx = ios::DeviceContext::get();
    return [&ctx](const ios::ConvProblem &p, int share) { return ctx.choose_launch(p, share); };
}

template <typename F>
int guarded(F &&body) {
    std::lock_guard<std::recursive_mutex> lock(g_api_mutex);
    try {
        body();
        return 0;
    } catch (const std::exception &e) {
        g_last_error = e.what();
    } catch (...) {
        g_last_error = "unknown error";
    }
    fprintf(stderr, "ios_runtime: %s\n", g_last_error.c_str());
    return 1;
}

int latency_call(ios::PlanMode mode, const char *doc_json, const char *extra_json, int batch_size, int warmup, int number,
                 int repeat, int profile_stage_latency, float *results, float *stage_results) {
    return guarded([&]() {
        if (results == nullptr) throw std::runtime_error("results pointer is null");
        const ios::Json doc = ios::Json::parse(doc_json);
        ios::Json extra;
        if (extra_json != nullptr) extra = ios::Json::parse(extra_json);
        ios::Plan plan = ios::build_plan(mode, doc, extra_json ? &extra : nullptr, batch_size, device_chooser());
        ios::Session session(std::move(plan), /*shared=*/true);
        if (mode == ios::PlanMode::Stage) {
            if (profile_stage_latency) throw std::runtime_error("stage_latency cannot profile stages (profile_stage_latency must be 0)");
            session.measure_back_to_back(warmup, number, repeat, results);
        } else {
            session.measure(warmup, number, repeat, profile_stage_latency != 0, results, stage_results);
        }
    });
}

struct SessionBox {
    std::unique_ptr<ios::Session> session;
    std::string description;
};

ios::Session &unbox(ios_session *s) {
    if (s == nullptr) throw std::runtime_error("session handle is null");
    return *reinterpret_cast<SessionBox *>(s)->session;
}

}  // namespace

extern "C" {

int graph_latency(const char *graph_json, int batch_size, int warmup, int number, int repeat, int profile_stage_latency,
                  float *results, float *stage_results) {
    return latency_call(ios::PlanMode::Graph, graph_json, nullptr, batch_size, warmup, number, repeat, profile_stage_latency, results,
                        stage_results);
}

int block_latency(const char *block_json, int batch_size, int warmup, int number, int repeat, int profile_stage_latency,
                  float *results, float *stage_results) {
    return latency_call(ios::PlanMode::Block, block_json, nullptr, batch_size, warmup, number, repeat, profile_stage_latency, results,
                        stage_results);
}

int stage_latency(const char *stage_json, const char *input_json, int batch_size, int warmup, int number, int repeat,
                  int profile_stage_latency, float *results, float *stage_results) {
    if (input_json == nullptr) input_json = "{}";
    return latency_call(ios::PlanMode::Stage, stage_json, input_json, batch_size, warmup, number, repeat, profile_stage_latency, results,
                        stage_results);
}

int graph_inference(const char *graph_json, int batch_size, float *input, int num_convs, char **conv_names, float **filter_data,
                    float **bias_data, float *output) {
    return guarded([&]() {
        const ios::Json doc = ios::Json::parse(graph_json);
        ios::Plan plan = ios::build_plan(ios::PlanMode::Graph, doc, nullptr, batch_size, device_chooser());
        ios::Session session(std::move(plan), /*shared=*/true);
        session.set_input(input);
        if (num_convs > 0 && (conv_names == nullptr || filter_data == nullptr || bias_data == nullptr))
            throw std::runtime_error("conv_names, filter_data or bias_data is null");
        for (int i = 0; i < num_convs; i++) session.set_conv_weights(conv_names[i], filter_data[i], bias_data[i]);
        session.run();
        session.get_output(output);
    });
}

int graph_inference_no_alloc(const char *graph_json, int batch_size, float *input, int num_convs, char **conv_names, float **filter_data,
                             float **bias_data, float *output) {
    return guarded([&]() {
        const ios::Json doc = ios::Json::parse(graph_json);
        ios::DeviceContext &ctx = ios::DeviceContext::get();
        // cached kernel configurations are used, missing ones are not measured (measuring allocates scratch tensors)
        ios::Plan plan = ios::build_plan(ios::PlanMode::Graph, doc, nullptr, batch_size,
                                         [&ctx](const ios::ConvProblem &p, int share) { return ctx.choose_launch(p, share, /*allow_tuning=*/false); });
        ios::Session session(std::move(plan), ios::Session::Storage::Static);
        session.set_input(input);
        if (num_convs > 0 && (conv_names == nullptr || filter_data == nullptr || bias_data == nullptr))
            throw std::runtime_error("conv_names, filter_data or bias_data is null");
        for (int i = 0; i < num_convs; i++) session.set_conv_weights(conv_names[i], filter_data[i], bias_data[i]);
        session.run();
        session.get_output(output);
    });
}

const char *ios_last_error(void) { return g_last_error.c_str(); }

int ios_set_option(const char *key, const char *value) {
    return guarded([&]() {
        if (key == nullptr || value == nullptr) throw std::runtime_error("option key or value is null");
        if (ios::set_planner_option(key, value)) return;   // needs no device
        ios::DeviceContext::get().set_option(key, value);
    });
}

int ios_device_info(char *buf, int cap) {
    return guarded([&]() {
        const std::string info = ios::DeviceContext::get().info_json();
        if (buf == nullptr || cap <= (int)info.size()) throw std::runtime_error("buffer too small");
        memcpy(buf, info.c_str(), info.size() + 1);
    });
}

long long ios_device_free_bytes(void) {
    long long bytes = -1;
    guarded([&]() {
        ios::DeviceContext::get();
        size_t free_bytes = 0, total = 0;
        if (hipMemGetInfo(&free_bytes, &total) != hipSuccess) throw std::runtime_error("hipMemGetInfo failed");
        bytes = (long long)free_bytes;
    });
    return bytes;
}

int ios_xcd_numbering(int tiles, int split, int *tile_of_block, int *slice_of_block, int capacity) {
    int blocks = -1;
    guarded([&]() {
        if (tiles < 1 || split < 1) throw std::runtime_error("xcd numbering: tiles >= 1 and split >= 1 required");
        blocks = ios::xcd_grid_blocks(tiles, split);
        if (tile_of_block == nullptr || slice_of_block == nullptr || capacity < blocks) return;
        const int q = tiles >> 3, r = tiles & 7;
        for (int b = 0; b < blocks; b++) {
            const ios::XcdSlot slot = ios::xcd_slot(b, (b >> 3) / split, q, r, split);
            // the tile a block works on, as the kernels derive it from the slot (xcd_tile)
            const int c = slot.tile & 7, in_class = slot.tile >> 3;
            tile_of_block[b] = slot.idle ? -1 : in_class + c * q + (c < r ? c : r);
            slice_of_block[b] = slot.slice;
        }
    });
    return blocks;
}

void ios_split_bf16x3(float x, unsigned *terms) {
    if (terms != nullptr) ios::split3(x, terms[0], terms[1], terms[2]);
}

int ios_conv_variant_names(char *buf, int cap) {
    std::string text = "[";
    for (int i = 0; i < ios::conv_num_variants(); i++) text += std::string(i ? "," : "") + '"' + ios::conv_variant(i).name + '"';
    text += "]";
    if (buf != nullptr && cap > (int)text.size()) memcpy(buf, text.c_str(), text.size() + 1);
    return (int)text.size();
}

// Kernel configurations of plans made without a device: the closed-form model for a 256-CU part.
static ios::LaunchChooser host_chooser() {
    return [](const ios::ConvProblem &p, int share) {
        ios::ConvLaunch launch = ios::conv_pick_launch(p, 256 / (share > 0 ? share : 1), share > 1);
        if (ios::planner_host_split_k() > 0) launch.split_k = ios::planner_host_split_k();
        return launch;
    };
}

int ios_plan_describe(const char *graph_json, int batch_size, char *buf, int cap) {
    int needed = -1;
    guarded([&]() {
        const ios::Json doc = ios::Json::parse(graph_json);
        // host-only: the closed-form configuration model for a 256-CU device, no device is touched
        ios::Plan plan = ios::build_plan(ios::PlanMode::Graph, doc, nullptr, batch_size,
                                         host_chooser());
        const std::string text = ios::describe_plan(plan);
        needed = (int)text.size();
        if (buf != nullptr && cap > needed) memcpy(buf, text.c_str(), text.size() + 1);
    });
    return needed;
}

long long ios_plan_arena_bytes(const char *graph_json, int batch_size) {
    long long bytes = -1;
    guarded([&]() {
        const ios::Json doc = ios::Json::parse(graph_json);
        ios::Plan plan = ios::build_plan(ios::PlanMode::Graph, doc, nullptr, batch_size,
                                         host_chooser());
        bytes = (long long)(plan.arena_floats * sizeof(float));
    });
    return bytes;
}

ios_session *ios_session_create(const char *graph_json, int batch_size) {
    SessionBox *box = nullptr;
    const int status = guarded([&]() {
        const ios::Json doc = ios::Json::parse(graph_json);
        ios::Plan plan = ios::build_plan(ios::PlanMode::Graph, doc, nullptr, batch_size, device_chooser());
        box = new SessionBox();
        box->description = ios::describe_plan(plan);
        box->session.reset(new ios::Session(std::move(plan), /*shared=*/false));
    });
    if (status != 0) {
        delete box;
        return nullptr;
    }
    return reinterpret_cast<ios_session *>(box);
}

void ios_session_destroy(ios_session *s) {
    if (s == nullptr) return;
    guarded([&]() { delete reinterpret_cast<SessionBox *>(s); });
}

int ios_session_set_conv_weights(ios_session *s, int num_convs, char **conv_names, float **filter_data, float **bias_data) {
    return guarded([&]() {
        ios::Session &session = unbox(s);
        if (num_convs > 0 && (conv_names == nullptr || filter_data == nullptr || bias_data == nullptr))
            throw std::runtime_error("conv_names, filter_data or bias_data is null");
        for (int i = 0; i < num_convs; i++) session.set_conv_weights(conv_names[i], filter_data[i], bias_data[i]);
    });
}

int ios_session_set_input(ios_session *s, const float *input) {
    return guarded([&]() { unbox(s).set_input(input); });
}

int ios_session_run(ios_session *s) {
    return guarded([&]() { unbox(s).run(); });
}

int ios_session_enqueue(ios_session *s) {
    return guarded([&]() { unbox(s).forward(); });
}

int ios_session_synchronize(ios_session *s) {
    return guarded([&]() { unbox(s).synchronize(); });
}

int ios_session_get_output(ios_session *s, float *output) {
    return guarded([&]() { unbox(s).get_output(output); });
}

int ios_session_get_tensor(ios_session *s, const char *node_name, float *output) {
    return guarded([&]() {
        if (node_name == nullptr || output == nullptr) throw std::runtime_error("null argument");
        unbox(s).get_tensor(node_name, output);
    });
}

int ios_session_measure(ios_session *s, int warmup, int number, int repeat, int profile_stage_latency, float *results,
                        float *stage_results) {
    return guarded([&]() {
        if (results == nullptr) throw std::runtime_error("results pointer is null");
        unbox(s).measure(warmup, number, repeat, profile_stage_latency != 0, results, stage_results);
    });
}

int ios_session_num_ops(ios_session *s) {
    int n = -1;
    guarded([&]() { n = (int)unbox(s).plan().ops.size(); });
    return n;
}

int ios_session_describe(ios_session *s, char *buf, int cap) {
    int needed = -1;
    guarded([&]() {
        unbox(s);
        const std::string &text = reinterpret_cast<SessionBox *>(s)->description;
        needed = (int)text.size();
        if (buf != nullptr && cap > needed) memcpy(buf, text.c_str(), text.size() + 1);
    });
    return needed;
}

int ios_session_profile_ops(ios_session *s, int warmup, int repeat, float *ms) {
    return guarded([&]() {
        if (ms == nullptr) throw std::runtime_error("output pointer is null");
        unbox(s).profile_ops(warmup, repeat, ms);
    });
}

int ios_session_describe_launches(ios_session *s, char *buf, int cap) {
    int needed = -1;
    guarded([&]() {
        const std::string text = unbox(s).describe_launches();
        needed = (int)text.size();
        if (buf != nullptr && cap > needed) memcpy(buf, text.c_str(), text.size() + 1);
    });
    return needed;
}

int ios_session_profile_launches(ios_session *s, int warmup, int repeat, float *ms, int capacity) {
    return guarded([&]() {
        if (ms == nullptr) throw std::runtime_error("output pointer is null");
        unbox(s).profile_launches(warmup, repeat, ms, capacity);
    });
}

}  // extern "C"
