// Execution plan: the flat list of device operations, tensor views and the memory layout that a graph,
// block or stage document compiles to.  Planning is pure host code; nothing here touches the device.
//
// Memory model: one arena of 4-byte words.  Every operator output, temporary, filter, bias and split-K
// workspace is a region of it at a 256-byte aligned offset.  Tensor views are
// (offset, C, H, W, batch stride); a channel slice or a window of a concat buffer is again a view, so
//   * an identity with one input value is an alias (no memory, no work),
//   * a producer whose whole output is one term of a concat writes directly into the concat buffer,
//   * a channel slice of a merged convolution is read in place at any batch size,
//   * a ReLU that only feeds the next convolution of its Sequential is folded into that convolution's
//     input loader.
#pragma once

#include <functional>
#include <map>
#include <set>
#include <string>
#include <vector>

#include "json.h"
#include "kernels.h"

namespace ios {

constexpr int kMaxGroups = 16;   // concurrent groups (streams) per stage
constexpr int kMaxExtent = 1 << 16;     // image sides, filter sides, strides and padding a document may ask for
constexpr int kMaxChannels = 1 << 20;   // channels of a tensor

struct ViewRef {
    size_t offset = 0;   // in floats from the arena base
    int C = 0, H = 0, W = 0;
    long long bstride = 0;
    ViewRef window(int begin, int end) const {
        ViewRef v = *this;
        v.offset += (size_t)begin * H * W;
        v.C = end - begin;
        return v;
    }
    size_t image_floats() const { return (size_t)C * H * W; }
};

enum class OpKind { ConvMfma, ConvDepthwise, ConvDirect, Pool, GlobalPool, Nary, Unary };
const char *op_kind_name(OpKind kind);

struct PlanConv {
    std::string name;
    ConvProblem problem;
    size_t weight_off = 0, bias_off = 0;       // original layouts
    size_t packed_off = 0;                     // matrix path only
    size_t ws_off = 0, ws_floats = 0;          // split-K only
    size_t ctr_off = 0, ctr_count = 0;         // split-K ticket counters (32-bit words at float offsets), zeroed at session setup
    ConvLaunch launch;
    bool matrix_path = false;
    // "average pool, then this convolution" run as "this convolution without bias and activation, then the pool, which adds
    // the bias and applies the activation": the convolution's launch reads OC zeros at zero_bias_off instead of the bias
    bool linear = false;
    size_t zero_bias_off = 0;
    bool thin = false;   // direct path: the kernel for 3 x 3 convolutions of 3-channel images (first layers at large batches)
};

struct PlanOp {
    OpKind kind;
    std::string node;     // operator name in the document
    int unit = -1;        // schedule unit (top-level operator) this op belongs to
    int stage = -1, group = -1;
    // position in the dependency order of the operations of its unit: operations of one unit on the same level are independent
    // of each other (the terms of a concatenation) and may run concurrently, a higher level reads what the lower ones wrote
    int level = 0;
    ViewRef in, out;
    int conv = -1;        // index into Plan::convs
    int bias_conv = -1;   // Pool behind a commuted convolution: out = act(pool(in) + bias of that convolution)
    PoolProblem pool{};
    std::vector<ViewRef> srcs;   // Nary: inputs; ConvDepthwise of a sum: the views it adds in its loader (else empty)
    int multiply = 0, accumulate = 0, act = 0;
    // ConvMfma of a residual unit: out = residual + act(conv + bias), then max(., 0) when post_relu
    bool has_residual = false;
    ViewRef residual;
    int post_relu = 0;
    double flops = 0.0, bytes = 0.0;
};

struct Plan {
    int batch = 1;
    std::vector<PlanOp> ops;
    std::vector<PlanConv> convs;
    std::vector<std::vector<std::vector<int>>> stages;   // stage -> group -> op indices in launch order
    std::vector<std::string> unit_names;
    std::map<std::string, ViewRef> tensors;              // operator name -> materialised output view
    std::map<std::string, int> conv_index;               // convolution name -> index into convs
    ViewRef input, output;
    std::string input_name, output_name;
    size_t arena_floats = 0;
    // layout of the arena: [0, persistent_floats) filters, biases, packed filters and split-K ticket counters, which live as
    // long as the plan; behind them the regions of operator outputs, temporaries and split-K partial tiles.  With reuse
    // (planner option "arena_reuse"), regions whose lifetimes (first to last stage that touches them) do not intersect share
    // addresses; `overwritten` names the operators whose output does not survive to the end of a pass for that reason.
    size_t persistent_floats = 0;
    size_t activation_floats_without_reuse = 0;
    std::set<std::string> overwritten;
    bool output_single_group = true;                     // the last stage has one group
};

enum class PlanMode { Graph, Block, Stage };

// Picks the kernel configuration of a matrix-path convolution (closed-form model or measured).  `share` is the
// number of groups that run concurrently in the convolution's stage: a kernel that shares the device with
// share - 1 others should occupy about 1 / share of it rather than all of it.
typedef std::function<ConvLaunch(const ConvProblem &, int share)> LaunchChooser;

// Compile a document.  `extra` is the input-shape document of stage mode ({name: [C, H, W]}).
// Throws std::runtime_error on malformed documents, unknown operator types, non-topological schedules
// and stages with too many groups.
Plan build_plan(PlanMode mode, const Json &doc, const Json *extra, int batch, const LaunchChooser &chooser);

std::string describe_plan(const Plan &plan);   // JSON array, one object per op

// Planner options that need no device: "arena_reuse" = "1" (default) | "0"; "thin_conv_min_pixels" = least number of output
// pixels (batch x OH x OW) from which a 3 x 3 convolution of a 3-channel image takes the output-bound direct kernel instead
// of the matrix path (default 2^18; a negative value disables it); "commute_pool_conv" = "1" (default) | "0": run "average
// pool that keeps the map size, then 1 x 1 convolution" as "convolution, then pool".  Returns false for an unknown key.
bool set_planner_option(const std::string &key, const std::string &value);
bool planner_arena_reuse();
long long planner_thin_conv_min_pixels();
int planner_host_split_k();   // option host_plan_split_k
bool planner_commute_pool_conv();   // option commute_pool_conv (default 1): see PlanConv::linear

}  // namespace ios
