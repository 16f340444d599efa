// Planner: JSON document -> Plan.  See plan.h for the memory model.  The document layout is the wire
// format exported by the Python IR (graph = {name, input, blocks}, block = {enter_name, enter_node,
// inner_nodes, exit_node, stages}, stage document = [[node config, ...] per group]); operator semantics
// are those the reference runtime gives the same documents (src/ios/ios_runtime.cu:1118-1240 for the
// three document kinds, :623-812 for the input algebra, :1047-1057 for pooling types).
#include "plan.h"

#include <climits>

#include <algorithm>
#include <cstdio>
#include <set>
#include <sstream>
#include <stdexcept>

namespace ios {

const char *op_kind_name(OpKind kind) {
    switch (kind) {
        case OpKind::ConvMfma: return "conv_mfma";
        case OpKind::ConvDepthwise: return "conv_depthwise";
        case OpKind::ConvDirect: return "conv_direct";
        case OpKind::Pool: return "pool";
        case OpKind::GlobalPool: return "global_pool";
        case OpKind::Nary: return "nary";
        case OpKind::Unary: return "unary";
    }
    return "?";
}

namespace {

struct Val {
    int node;
    int begin, end;
};

enum class NodeType { Placeholder, Conv, Pool, Identity, Relu, Activation, Element, Sequential };

struct PNode {
    std::string name;
    NodeType type = NodeType::Placeholder;
    const Json *cfg = nullptr;
    int C = 0, H = 0, W = 0;
    std::vector<std::vector<Val>> inputs;
    int unit = -1;
    // storage: either an own region or a channel window of another node's storage
    bool own = false;
    size_t own_offset = 0;
    int parent = -1, parent_begin = 0;
    bool pre_relu_alias = false;   // elided ReLU: consumers must apply max(x, 0) themselves
    int fused_into = -1;           // concat (identity) node whose buffer holds this node's output
    bool no_storage = false;       // ReLU whose inputs the consumer reads itself: never materialised
    // depth-wise convolution that adds the values of a sum in its loader: the node whose single term
    // holds them (the convolution itself, or the private ReLU in front of it, which is then applied after the sum)
    int sum_front = -1;
    bool sum_relu = false;
    int combine_front = -1;        // activation that combines the values of this addition / product / sum itself
    // Residual unit: a convolution whose only reader is an addition with one other value adds that value in its epilogue and
    // writes the addition's tensor (or that of the ReLU absorbing the addition).  On the convolution: the node whose storage
    // it writes, the other value and the ReLU; on that node: made_by_conv.
    int residual_into = -1;
    Val residual_other{-1, 0, 0};
    bool residual_relu = false;
    bool made_by_conv = false;
    // "average pool, then 1 x 1 convolution" run as "1 x 1 convolution, then average pool": on the pool the convolution, on
    // the convolution the pool
    int commuted_conv = -1, commuted_pool = -1;
    int references = 0;            // number of input values that name this node
};

int act_code(const std::string &name) {
    if (name == "identity") return ACT_NONE;
    if (name == "relu") return ACT_RELU;
    if (name == "tanh") return ACT_TANH;
    if (name == "sigmoid") return ACT_SIGMOID;
    throw std::runtime_error("unsupported activation '" + name + "'");
}

class Planner {
public:
    Planner(int batch, const LaunchChooser &chooser) : batch_(batch), chooser_(chooser) {
        if (batch < 1) throw std::runtime_error("batch size must be positive");
        plan_.batch = batch;
    }

    Plan run(PlanMode mode, const Json &doc, const Json *extra) {
        std::vector<std::vector<std::vector<std::string>>> stage_names;
        if (mode == PlanMode::Graph) {
            add_placeholder(doc["input"]["name"].as_string(), doc["input"]["output_shape"]);
            plan_.input_name = nodes_[0].name;
            for (const Json &block : doc["blocks"].items()) add_block(block, stage_names);
        } else if (mode == PlanMode::Block) {
            const Json &enter = doc["enter_node"];
            add_placeholder(enter["name"].as_string(), enter["output_shape"]);
            plan_.input_name = nodes_[0].name;
            add_block(doc, stage_names);
        } else {
            if (extra == nullptr || !extra->is_object()) throw std::runtime_error("stage document needs an input-shape document");
            for (const auto &member : extra->members()) add_placeholder(member.first, member.second);
            if (!doc.is_array() || doc.size() == 0) throw std::runtime_error("stage document must be a non-empty list of groups");
            std::vector<std::vector<std::string>> groups;
            for (const Json &group : doc.items()) {
                std::vector<std::string> names;
                for (const Json &cfg : group.items()) {
                    add_unit(cfg);
                    names.push_back(cfg["name"].as_string());
                }
                groups.push_back(names);
            }
            stage_names.push_back(groups);
            if (!nodes_.empty() && nodes_[0].type == NodeType::Placeholder) plan_.input_name = nodes_[0].name;
        }
        if (units_.empty()) throw std::runtime_error("document contains no operators");
        index_schedule(stage_names);
        decide_storage();
        allocate_outputs();
        for (size_t i = 0; i < nodes_.size(); i++) emit(static_cast<int>(i));
        assign_stages(stage_names);
        finish();
        return std::move(plan_);
    }

private:
    // ---- document -> node table ---------------------------------------------------------------------------
    int lookup(const std::string &name) const {
        auto it = by_name_.find(name);
        if (it == by_name_.end()) throw std::runtime_error("operator '" + name + "' is used before it is defined");
        return it->second;
    }

    void add_placeholder(const std::string &name, const Json &shape) {
        if (by_name_.count(name)) throw std::runtime_error("duplicate operator name '" + name + "'");
        PNode n;
        n.name = name;
        n.type = NodeType::Placeholder;
        n.C = shape[0].as_int();
        n.H = shape[1].as_int();
        n.W = shape[2].as_int();
        if (n.C < 1 || n.H < 1 || n.W < 1 || n.C > kMaxChannels || n.H > kMaxExtent || n.W > kMaxExtent)
            throw std::runtime_error("placeholder '" + name + "': bad shape");
        n.own = true;
        by_name_[name] = static_cast<int>(nodes_.size());
        nodes_.push_back(n);
    }

    void add_block(const Json &block, std::vector<std::vector<std::vector<std::string>>> &stage_names) {
        for (const Json &cfg : block["inner_nodes"].items()) add_unit(cfg);
        add_unit(block["exit_node"]);
        const Json &stages = block["stages"];
        if (!stages.is_array()) throw std::runtime_error("block has no schedule (stages is null); call sequential_schedule() first");
        for (const Json &stage : stages.items()) {
            std::vector<std::vector<std::string>> groups;
            for (const Json &group : stage.items()) {
                std::vector<std::string> names;
                for (const Json &name : group.items()) names.push_back(name.as_string());
                groups.push_back(names);
            }
            stage_names.push_back(groups);
        }
    }

    void add_unit(const Json &cfg) {
        const int unit = static_cast<int>(units_.size());
        units_.push_back(cfg["name"].as_string());
        plan_.unit_names.push_back(units_.back());
        const int index = add_node(cfg, unit);
        unit_result_.push_back(index);
    }

    std::vector<std::vector<Val>> parse_inputs(const Json &inputs) {
        std::vector<std::vector<Val>> terms;
        for (const Json &term : inputs.items()) {
            std::vector<Val> values;
            for (const Json &value : term.items()) {
                Val v{lookup(value[0].as_string()), value[1].as_int(), value[2].as_int()};
                const PNode &src = nodes_[v.node];
                if (v.begin < 0 || v.end > src.C || v.begin >= v.end)
                    throw std::runtime_error("bad channel slice of '" + src.name + "'");
                nodes_[v.node].references++;
                values.push_back(v);
            }
            if (values.empty()) throw std::runtime_error("empty input term");
            terms.push_back(values);
        }
        if (terms.empty()) throw std::runtime_error("operator without inputs");
        return terms;
    }

    void input_shape(const PNode &n, int &C, int &H, int &W) const {
        C = 0;
        H = nodes_[n.inputs[0][0].node].H;
        W = nodes_[n.inputs[0][0].node].W;
        for (const auto &term : n.inputs) {
            const int len = term[0].end - term[0].begin;
            for (const Val &v : term) {
                if (v.end - v.begin != len || nodes_[v.node].H != H || nodes_[v.node].W != W)
                    throw std::runtime_error("operator '" + n.name + "': input values of different shapes");
            }
            C += len;
        }
    }

    int add_node(const Json &cfg, int unit) {
        const std::string type = cfg["type"].as_string();
        const std::string name = cfg["name"].as_string();
        if (by_name_.count(name)) throw std::runtime_error("duplicate operator name '" + name + "'");
        if (type == "sequential") {
            const Json &children = cfg["nodes"];
            if (children.size() == 0) throw std::runtime_error("empty sequential operator '" + name + "'");
            int last = -1;
            const int first_child = static_cast<int>(nodes_.size());
            for (const Json &child : children.items()) last = add_node(child, unit);
            sequentials_.push_back({first_child, last});
            PNode n;
            n.name = name;
            n.type = NodeType::Sequential;
            n.cfg = &cfg;
            n.unit = unit;
            n.C = nodes_[last].C;
            n.H = nodes_[last].H;
            n.W = nodes_[last].W;
            n.parent = last;
            by_name_[name] = static_cast<int>(nodes_.size());
            nodes_.push_back(n);
            return static_cast<int>(nodes_.size()) - 1;
        }
        PNode n;
        n.name = name;
        n.cfg = &cfg;
        n.unit = unit;
        n.inputs = parse_inputs(cfg["inputs"]);
        int C, H, W;
        input_shape(n, C, H, W);
        if (type == "conv") {
            n.type = NodeType::Conv;
            const int kh = cfg["kernel"][0].as_int(), kw = cfg["kernel"][1].as_int();
            const int sh = cfg["stride"][0].as_int(), sw = cfg["stride"][1].as_int();
            const int ph = cfg["padding"][0].as_int(), pw = cfg["padding"][1].as_int();
            const int groups = cfg["groups"].as_int();
            n.C = cfg["out_channels"].as_int();
            if (groups < 1 || C % groups != 0 || n.C % groups != 0)
                throw std::runtime_error("conv '" + name + "': channels not divisible by groups");
            if (sh < 1 || sw < 1 || kh < 1 || kw < 1 || ph < 0 || pw < 0 || std::max({kh, kw, sh, sw, ph, pw}) > kMaxExtent)
                throw std::runtime_error("conv '" + name + "': bad geometry");
            if (n.C < 1 || n.C > kMaxChannels) throw std::runtime_error("conv '" + name + "': bad channel count");
            // C++ division truncates towards zero: a window larger than the padded input would come out as one output row
            if (H + 2 * ph < kh || W + 2 * pw < kw) throw std::runtime_error("conv '" + name + "': kernel larger than the padded input");
            n.H = 1 + (H - kh + 2 * ph) / sh;
            n.W = 1 + (W - kw + 2 * pw) / sw;
            act_code(cfg["act"].as_string());
        } else if (type == "pool") {
            n.type = NodeType::Pool;
            n.C = C;
            const std::string pool_type = cfg["pool_type"].as_string();
            // the reference only looks for the substrings "max" and "global" and takes everything else for an average
            // (src/ios/ios_runtime.cu:1047-1051; its AlexNet writes 'max_pool'); a name with neither "max" nor "avg" is
            // refused here instead of silently averaging
            if (pool_type.find("max") == std::string::npos && pool_type.find("avg") == std::string::npos)
                throw std::runtime_error("pool '" + name + "': unknown pool_type '" + pool_type + "'");
            if (pool_type.find("global") != std::string::npos) {
                n.H = 1;
                n.W = 1;
            } else {
                const int kh = cfg["kernel"][0].as_int(), kw = cfg["kernel"][1].as_int();
                const int sh = cfg["stride"][0].as_int(), sw = cfg["stride"][1].as_int();
                const int ph = cfg["padding"][0].as_int(), pw = cfg["padding"][1].as_int();
                if (sh < 1 || sw < 1 || kh < 1 || kw < 1 || ph < 0 || pw < 0 || std::max({kh, kw, sh, sw, ph, pw}) > kMaxExtent)
                    throw std::runtime_error("pool '" + name + "': bad geometry");
                if (H + 2 * ph < kh || W + 2 * pw < kw) throw std::runtime_error("pool '" + name + "': window larger than the padded input");
                n.H = 1 + (H - kh + 2 * ph) / sh;
                n.W = 1 + (W - kw + 2 * pw) / sw;
            }
        } else if (type == "identity" || type == "relu" || type == "activation" || type == "element") {
            n.type = type == "identity" ? NodeType::Identity
                     : type == "relu"   ? NodeType::Relu
                     : type == "activation" ? NodeType::Activation
                                            : NodeType::Element;
            if (n.type == NodeType::Element) {
                if (n.inputs.size() != 1) throw std::runtime_error("element '" + name + "' needs exactly one term");
                const std::string op = cfg["op_type"].as_string();
                if (op != "add" && op != "mul") throw std::runtime_error("element '" + name + "': unknown op_type " + op);
            }
            if (n.type == NodeType::Activation) act_code(cfg["act_type"].as_string());
            n.C = C;
            n.H = H;
            n.W = W;
        } else {
            throw std::runtime_error("unsupported type " + type);
        }
        if (n.H < 1 || n.W < 1) throw std::runtime_error("operator '" + name + "' has an empty output");
        by_name_[name] = static_cast<int>(nodes_.size());
        nodes_.push_back(n);
        return static_cast<int>(nodes_.size()) - 1;
    }

    // ---- storage decisions -----------------------------------------------------------------------------------
    static bool single_value(const PNode &n) { return n.inputs.size() == 1 && n.inputs[0].size() == 1; }

    bool computes_own_output(const PNode &n) const {
        switch (n.type) {
            case NodeType::Conv:
            case NodeType::Pool:
            case NodeType::Element: return true;
            case NodeType::Relu:
            case NodeType::Activation: return !n.pre_relu_alias;
            case NodeType::Identity: return !single_value(n);
            default: return false;
        }
    }

    void decide_storage() {
        // ReLU directly in front of a convolution inside one Sequential, read by nobody else: fold it
        for (const auto &seq : sequentials_) {
            for (int i = seq.first; i < seq.second; i++) {
                PNode &r = nodes_[i];
                const PNode &next = nodes_[i + 1];
                if (r.type == NodeType::Relu && next.type == NodeType::Conv && single_value(r) && r.references == 1 &&
                    single_value(next) && next.inputs[0][0].node == i) {
                    r.pre_relu_alias = true;
                    r.parent = r.inputs[0][0].node;
                    r.parent_begin = r.inputs[0][0].begin;
                }
            }
        }
        find_depthwise_sums();
        find_activated_combinations();
        find_residual_convolutions();
        find_commuting_pools();
        for (PNode &n : nodes_) {
            if (n.type == NodeType::Identity && single_value(n)) {
                n.parent = n.inputs[0][0].node;
                n.parent_begin = n.inputs[0][0].begin;
            }
        }
        // concat fusion: a term that is the whole output of a computing operator is produced in place
        for (size_t i = 0; i < nodes_.size(); i++) {
            PNode &cat = nodes_[i];
            if (cat.type != NodeType::Identity || cat.inputs.size() < 2) continue;
            int offset = 0;
            for (const auto &term : cat.inputs) {
                const int len = term[0].end - term[0].begin;
                if (term.size() == 1) {
                    const int src = resolve_sequential(term[0].node);
                    PNode &p = nodes_[src];
                    if (term[0].begin == 0 && term[0].end == p.C && computes_own_output(p) && p.fused_into < 0 &&
                        p.parent < 0) {
                        p.fused_into = static_cast<int>(i);
                        p.parent = static_cast<int>(i);
                        p.parent_begin = offset;
                    }
                }
                offset += len;
            }
        }
        for (PNode &n : nodes_)
            if (n.parent < 0 && !n.no_storage) n.own = true;
    }

    ConvProblem problem_of(const PNode &n) const {
        int C, H, W;
        input_shape(n, C, H, W);
        const Json &cfg = *n.cfg;
        ConvProblem p;
        p.B = batch_;
        p.IC = C; p.H = H; p.W = W;
        p.OC = n.C; p.OH = n.H; p.OW = n.W;
        p.KH = cfg["kernel"][0].as_int(); p.KW = cfg["kernel"][1].as_int();
        p.sh = cfg["stride"][0].as_int(); p.sw = cfg["stride"][1].as_int();
        p.ph = cfg["padding"][0].as_int(); p.pw = cfg["padding"][1].as_int();
        p.groups = cfg["groups"].as_int();
        p.act = act_code(cfg["act"].as_string());
        p.pre_relu = 0;
        return p;
    }

    // Sequential children [(ReLU,) depth-wise K x K convolution, ...] whose input is one term that sums k > 1 values, read by
    // nobody else: the depth-wise kernel adds the k values (and applies the ReLU) in its loader, so the summing launch and its
    // output tensor disappear (the reference adds them with a kernel of its own, src/ios/ios_runtime.cu:1047-1057).
    void find_depthwise_sums() {
        // The summing loader addresses every source with 31-bit byte offsets.  Where the sources will live is decided later
        // (a source may become a window of a wider concatenation buffer), so the test assumes the widest tensor of the graph
        // as the batch stride; a sum that could exceed the range keeps its own launch and the generic depth-wise path.
        unsigned long long widest = 0;
        for (const PNode &n : nodes_) widest = std::max(widest, (unsigned long long)n.C * n.H * n.W);
        for (const auto &seq : sequentials_) {
            for (int i = seq.first; i <= seq.second; i++) {
                PNode &dw = nodes_[i];
                if (dw.type != NodeType::Conv) continue;
                const ConvProblem pd = problem_of(dw);
                if (!pd.is_depthwise() || !dwconv_sums_inputs(pd)) continue;
                int front = i;   // node whose inputs are the sources
                bool relu = false;
                if (single_value(dw) && i > seq.first && dw.inputs[0][0].node == i - 1) {
                    const PNode &r = nodes_[i - 1];
                    const bool whole = dw.inputs[0][0].begin == 0 && dw.inputs[0][0].end == r.C;
                    if (r.type == NodeType::Relu && r.references == 1 && whole && r.inputs.size() == 1) {
                        front = i - 1;
                        relu = true;
                    }
                }
                const PNode &f = nodes_[front];
                if (f.inputs.size() != 1 || f.inputs[0].size() < 2 || f.inputs[0].size() > (size_t)kMaxNaryInputs) continue;
                if (((unsigned long long)(batch_ - 1) * widest + (unsigned long long)pd.IC * pd.H * pd.W) * 4ull >= (1ull << 31)) continue;
                dw.sum_front = front;
                dw.sum_relu = relu;
                if (front != i) {
                    PNode &r = nodes_[front];
                    r.no_storage = true;   // the convolution reads the ReLU's inputs itself
                    r.parent = -1;
                }
            }
        }
    }

    // An activation whose only input is the whole output of an addition, a product or a sum of values that nobody else
    // reads (the residual unit "add, then ReLU" of reference python/ios/models/resnet.py:25-26): the activation's launch
    // combines the values itself, so the combining launch and its tensor disappear (the reference runs both,
    // src/ios/ios_runtime.cu:854-908,939-1010).
    void find_activated_combinations() {
        for (PNode &a : nodes_) {
            if ((a.type != NodeType::Relu && a.type != NodeType::Activation) || !single_value(a) || a.pre_relu_alias || a.no_storage)
                continue;
            const Val &v = a.inputs[0][0];
            PNode &e = nodes_[v.node];
            const bool combines = e.type == NodeType::Element || (e.type == NodeType::Identity && e.inputs.size() == 1 && e.inputs[0].size() >= 2);
            if (!combines || e.inputs.size() != 1 || e.inputs[0].size() > (size_t)kMaxNaryInputs) continue;
            if (e.references != 1 || e.no_storage || v.begin != 0 || v.end != e.C) continue;
            a.combine_front = v.node;
            e.no_storage = true;
        }
    }

    // Where the schedule puts every unit (names the schedule does not know stay at -1; assign_stages reports them).
    void index_schedule(const std::vector<std::vector<std::vector<std::string>>> &stage_names) {
        std::map<std::string, int> unit_of;
        for (size_t u = 0; u < units_.size(); u++) unit_of[units_[u]] = static_cast<int>(u);
        slots_.assign(units_.size(), Slot{});
        groups_in_stage_.clear();
        for (const auto &stage : stage_names) groups_in_stage_.push_back((int)stage.size());
        for (size_t s = 0; s < stage_names.size(); s++)
            for (size_t g = 0; g < stage_names[s].size(); g++)
                for (size_t k = 0; k < stage_names[s][g].size(); k++) {
                    auto it = unit_of.find(stage_names[s][g][k]);
                    if (it != unit_of.end()) slots_[it->second] = Slot{(int)s, (int)g, (int)k};
                }
    }

    bool alone_in_its_stage(int unit) const { return slots_[unit].stage >= 0 && groups_in_stage_[slots_[unit].stage] == 1; }

    // true when everything `node` writes is complete before the unit `consumer_unit` starts
    bool complete_before(int node, int consumer_unit) const {
        const int unit = nodes_[node].unit;
        if (unit < 0) return true;   // placeholder
        const Slot &a = slots_[unit], &b = slots_[consumer_unit];
        if (a.stage < 0 || b.stage < 0) return false;
        return a.stage < b.stage || (a.stage == b.stage && a.group == b.group && a.pos < b.pos);
    }

    // "convolution, + skip value (, ReLU)" of a residual unit (reference python/ios/models/resnet.py:10-27): when the
    // convolution's output is read by the addition only, the skip value is complete before the convolution starts, the
    // convolution has its stage to itself and takes the matrix path, its epilogue adds the skip value (and applies the
    // ReLU) and the addition's launch and the convolution's own tensor disappear.  The rounding is that of the separate
    // launches: act(conv + bias) is rounded to fp32 before the skip value is added.
    void find_residual_convolutions() {
        for (size_t i = 0; i < nodes_.size(); i++) {
            PNode &e = nodes_[i];
            if (e.type != NodeType::Element || (*e.cfg)["op_type"].as_string() != "add") continue;
            if (e.inputs.size() != 1 || e.inputs[0].size() != 2 || e.made_by_conv) continue;
            // the node that holds the result: the addition, or the activation that absorbed it
            int holder = static_cast<int>(i);
            bool relu = false;
            if (e.no_storage) {
                holder = -1;
                for (size_t k = 0; k < nodes_.size(); k++)
                    if (nodes_[k].combine_front == static_cast<int>(i)) holder = static_cast<int>(k);
                if (holder < 0) continue;
                const PNode &act = nodes_[holder];
                const int code = act.type == NodeType::Relu ? ACT_RELU : act_code((*act.cfg)["act_type"].as_string());
                if (code != ACT_RELU) continue;
                relu = true;
            }
            for (int side = 0; side < 2; side++) {
                const Val &mine = e.inputs[0][side], &other = e.inputs[0][1 - side];
                PNode &c = nodes_[mine.node];
                if (c.type != NodeType::Conv || c.unit < 0 || c.references != 1 || mine.begin != 0 || mine.end != c.C) continue;
                if (c.residual_into >= 0 || c.sum_front >= 0 || nodes_[other.node].type == NodeType::Sequential) continue;
                if (unit_result_[c.unit] != mine.node) continue;   // a member of a Sequential
                const ConvProblem p = problem_of(c);
                if (p.is_depthwise() || (p.groups > 1 && (p.ICg() < 4 || p.OCg() < 8)) || !conv_matrix_path_supported(p) || conv_thin_applies(p))
                    continue;
                if ((unsigned long long)batch_ * p.OC * p.OH * p.OW * 4ull >= (1ull << 30)) continue;
                // (the residual epilogue exists in the stand-alone kernels only: a stage of several groups is one fused launch)
                if (!alone_in_its_stage(c.unit) || !complete_before(other.node, c.unit)) continue;
                c.residual_into = holder;
                c.parent = holder;   // the convolution writes the holder's tensor
                c.parent_begin = 0;
                c.residual_other = other;
                c.residual_relu = relu;
                nodes_[holder].made_by_conv = true;
                if (holder != static_cast<int>(i)) nodes_[holder].combine_front = -1;   // nothing left to combine
                e.no_storage = holder != static_cast<int>(i);
                break;
            }
        }
    }

    // "Average pool that keeps the map size, then 1 x 1 convolution to no more channels, read by nobody else" (the pool branch
    // of the reference's Inception blocks, python/ios/models/inception_v3.py:28-29,62-63,96-97; pool semantics
    // src/ios/ios_runtime.cu:542-550, average over the padded window): both are linear and act on different axes, so W * pool(x) = pool(W * x) with the same
    // border rule.  The launch at the pool's place in the schedule computes z = W * x (no bias, no activation), the launch at
    // the convolution's place pools z, adds the bias and applies the activation: the pool then moves OC instead of IC
    // channels, and the pooled input tensor is neither written nor read back.  Sums are rounded in another order than in the
    // reference's sequence of operators (differences of a few units in the last place).
    void find_commuting_pools() {
        if (!planner_commute_pool_conv()) return;
        for (size_t i = 0; i < nodes_.size(); i++) {
            PNode &c = nodes_[i];
            if (c.type != NodeType::Conv || !single_value(c) || c.sum_front >= 0 || c.residual_into >= 0) continue;
            const Val &v = c.inputs[0][0];
            PNode &pool = nodes_[v.node];
            if (pool.type != NodeType::Pool || v.begin != 0 || v.end != pool.C || pool.references != 1 || !single_value(pool)) continue;
            bool wrapped = false;   // the result of a Sequential can be read under the Sequential's name
            for (const PNode &s : nodes_) wrapped = wrapped || (s.type == NodeType::Sequential && s.parent == v.node);
            if (wrapped || pool.no_storage || pool.commuted_conv >= 0) continue;
            const std::string pool_type = (*pool.cfg)["pool_type"].as_string();
            if (pool_type.find("avg") == std::string::npos || pool_type.find("max") != std::string::npos ||
                pool_type.find("global") != std::string::npos)
                continue;
            const PNode &x = nodes_[pool.inputs[0][0].node];
            if (x.pre_relu_alias || x.H != pool.H || x.W != pool.W) continue;
            const ConvProblem p = problem_of(c);
            if (p.KH != 1 || p.KW != 1 || p.sh != 1 || p.sw != 1 || p.ph != 0 || p.pw != 0 || p.groups != 1 || p.OC > p.IC) continue;
            if (!conv_matrix_path_supported(p) || conv_thin_applies(p)) continue;
            pool.commuted_conv = static_cast<int>(i);
            pool.no_storage = true;   // z lives in a temporary of the convolution's channel count
            pool.parent = -1;
            c.commuted_pool = v.node;
        }
    }

    int resolve_sequential(int index) const {
        while (nodes_[index].type == NodeType::Sequential) index = nodes_[index].parent;
        return index;
    }

    // persistent storage (filters, biases, packed filters, ticket counters): final offsets, handed out front to back
    size_t reserve(size_t floats) {
        const size_t at = plan_.arena_floats;
        plan_.arena_floats += (floats + 63) & ~size_t(63);
        return at;
    }

    // Storage with a lifetime (operator outputs, temporaries, split-K partial tiles): a region in a virtual address space,
    // marked by kRegionTag in its offsets, that place_regions() maps behind the persistent storage once the stages are known.
    static constexpr size_t kRegionTag = size_t(1) << 62;
    struct Region {
        size_t voff, floats;
        int first = INT_MAX, last = -1;   // stages that touch it
        bool pinned = false;              // lives for the whole pass (inputs, the result)
        size_t at = 0;                    // final offset
    };
    size_t reserve_region(size_t floats, bool pinned = false) {
        Region r;
        r.voff = region_floats_;
        r.floats = (std::max<size_t>(floats, 1) + 63) & ~size_t(63);
        r.pinned = pinned;
        region_floats_ += r.floats;
        regions_.push_back(r);
        return r.voff | kRegionTag;
    }
    Region *region_of(size_t offset) {
        if (!(offset & kRegionTag)) return nullptr;
        const size_t v = offset & ~kRegionTag;
        auto it = std::upper_bound(regions_.begin(), regions_.end(), v, [](size_t value, const Region &r) { return value < r.voff; });
        if (it == regions_.begin()) throw std::runtime_error("internal: view outside every region");
        --it;
        if (v >= it->voff + it->floats) throw std::runtime_error("internal: view outside its region");
        return &*it;
    }
    void touch(size_t offset, int stage) {
        if (Region *r = region_of(offset)) {
            r->first = std::min(r->first, stage);
            r->last = std::max(r->last, stage);
        }
    }
    size_t placed(size_t offset) {
        Region *r = region_of(offset);
        return r ? r->at + ((offset & ~kRegionTag) - r->voff) : offset;
    }

    // Lifetimes from the stages of the operations that read or write a region; then first-fit placement, largest regions
    // first, where two regions may share addresses when their lifetimes do not intersect (all operations of a stage have
    // finished before the next stage starts, under every executor); finally every offset of the plan is rewritten.
    void place_regions() {
        const int last_stage = (int)plan_.stages.size() - 1;
        for (const PlanOp &op : plan_.ops) {
            touch(op.in.offset, op.stage);
            touch(op.out.offset, op.stage);
            for (const ViewRef &v : op.srcs) touch(v.offset, op.stage);
            if (op.has_residual) touch(op.residual.offset, op.stage);
            if (op.conv >= 0 && plan_.convs[op.conv].ws_floats > 0) touch(plan_.convs[op.conv].ws_off, op.stage);
        }
        if (Region *r = region_of(plan_.output.offset)) r->pinned = true;
        const bool reuse = planner_arena_reuse();
        for (Region &r : regions_)
            if (r.pinned || !reuse || r.last < 0) {   // (an untouched region belongs to an operator nobody reads: keep it apart)
                r.first = 0;
                r.last = last_stage;
            }
        std::vector<Region *> order;
        for (Region &r : regions_) order.push_back(&r);
        std::stable_sort(order.begin(), order.end(), [](const Region *a, const Region *b) { return a->floats > b->floats; });
        std::vector<Region *> done;
        size_t extent = 0;
        for (Region *r : order) {
            // candidate offsets: 0 and the end of every placed region that is alive at the same time
            std::vector<std::pair<size_t, size_t>> busy;   // [begin, end) of conflicting regions
            for (Region *o : done)
                if (o->first <= r->last && r->first <= o->last) busy.push_back({o->at, o->at + o->floats});
            std::sort(busy.begin(), busy.end());
            size_t at = 0;
            for (const auto &b : busy) {
                if (at + r->floats <= b.first) break;
                at = std::max(at, b.second);
            }
            r->at = at;
            extent = std::max(extent, at + r->floats);
            done.push_back(r);
        }
        const size_t base = plan_.arena_floats;
        plan_.persistent_floats = base;
        plan_.activation_floats_without_reuse = region_floats_;
        for (Region &r : regions_) r.at += base;
        // (the vectorised pooling kernel reads up to eight floats past the end of a tensor and discards them: the arena ends
        // in padding so that such a read stays inside the allocation)
        plan_.arena_floats = base + extent + 64;
        // names of the outputs that a later region overwrites
        for (auto &entry : plan_.tensors) {
            const Region *r = region_of(entry.second.offset);
            if (r == nullptr) continue;
            for (const Region &o : regions_)
                if (&o != r && o.first > r->last && o.at < r->at + r->floats && r->at < o.at + o.floats) {
                    plan_.overwritten.insert(entry.first);
                    break;
                }
        }
        for (PlanOp &op : plan_.ops) {
            op.in.offset = placed(op.in.offset);
            op.out.offset = placed(op.out.offset);
            for (ViewRef &v : op.srcs) v.offset = placed(v.offset);
            if (op.has_residual) op.residual.offset = placed(op.residual.offset);
        }
        for (PlanConv &c : plan_.convs)
            if (c.ws_floats > 0) c.ws_off = placed(c.ws_off);
        for (auto &entry : plan_.tensors) entry.second.offset = placed(entry.second.offset);
        plan_.input.offset = placed(plan_.input.offset);
        plan_.output.offset = placed(plan_.output.offset);
    }

    void allocate_outputs() {
        for (PNode &n : nodes_)
            if (n.own) n.own_offset = reserve_region((size_t)batch_ * n.C * n.H * n.W, /*pinned=*/n.type == NodeType::Placeholder);
    }

    ViewRef view_of(int index) const {
        const PNode &n = nodes_[index];
        if (n.own) {
            ViewRef v;
            v.offset = n.own_offset;
            v.C = n.C;
            v.H = n.H;
            v.W = n.W;
            v.bstride = (long long)n.C * n.H * n.W;
            return v;
        }
        return view_of(n.parent).window(n.parent_begin, n.parent_begin + n.C);
    }

    bool needs_relu(int index) const {
        // true when the value seen through `index` is an elided ReLU (possibly behind aliases)
        const PNode &n = nodes_[index];
        if (n.pre_relu_alias) return true;
        return false;
    }

    ViewRef dense_temp(int C, int H, int W) {
        ViewRef v;
        v.offset = reserve_region((size_t)batch_ * C * H * W);
        v.C = C;
        v.H = H;
        v.W = W;
        v.bstride = (long long)C * H * W;
        return v;
    }

    // ---- op emission --------------------------------------------------------------------------------------------
    PlanOp &push(OpKind kind, const PNode &owner) {
        PlanOp op;
        op.kind = kind;
        op.node = owner.name;
        op.unit = owner.unit;
        op.level = level_base_;
        level_top_ = std::max(level_top_, op.level + 1);
        plan_.ops.push_back(op);
        return plan_.ops.back();
    }

    // dst = act(combine(values of term)); dst has the term's channel count
    void materialise_term(const PNode &owner, const std::vector<Val> &term, const ViewRef &dst, int act, bool multiply) {
        const double elems = (double)batch_ * dst.image_floats();
        if (term.size() == 1) {
            PlanOp &op = push(OpKind::Unary, owner);
            op.in = view_of(term[0].node).window(term[0].begin, term[0].end);
            op.out = dst;
            op.act = act;
            op.bytes = 8.0 * elems;
            return;
        }
        for (size_t first = 0; first < term.size(); first += kMaxNaryInputs) {
            const size_t last = std::min(term.size(), first + kMaxNaryInputs);
            PlanOp &op = push(OpKind::Nary, owner);
            for (size_t i = first; i < last; i++) op.srcs.push_back(view_of(term[i].node).window(term[i].begin, term[i].end));
            op.out = dst;
            op.multiply = multiply ? 1 : 0;
            op.accumulate = first > 0 ? 1 : 0;
            op.act = last == term.size() ? act : ACT_NONE;
            op.flops = elems * (double)(last - first - (first > 0 ? 0 : 1));
            op.bytes = 4.0 * elems * (double)(last - first + 1 + (first > 0 ? 1 : 0));
            op.level = level_base_ + (int)(first / kMaxNaryInputs);   // accumulation chunks of one term follow each other
            level_top_ = std::max(level_top_, op.level + 1);
        }
    }

    // the operator's input as one view; builds it in a temporary when it is a sum or a concatenation
    ViewRef input_view(const PNode &n, int C, int H, int W, bool *pre_relu) {
        if (pre_relu) *pre_relu = false;
        if (single_value(n)) {
            const Val &v = n.inputs[0][0];
            if (nodes_[v.node].pre_relu_alias) {
                if (pre_relu == nullptr) throw std::runtime_error("internal: folded ReLU read by a non-convolution");
                *pre_relu = true;
            }
            return view_of(v.node).window(v.begin, v.end);
        }
        ViewRef temp = dense_temp(C, H, W);
        int offset = 0;
        for (const auto &term : n.inputs) {
            const int len = term[0].end - term[0].begin;
            materialise_term(n, term, temp.window(offset, offset + len), ACT_NONE, false);
            offset += len;
        }
        level_base_ = level_top_;   // the operator itself reads what the terms wrote
        return temp;
    }

    void emit(int index) {
        PNode &n = nodes_[index];
        if (n.type == NodeType::Placeholder || n.type == NodeType::Sequential) return;
        if (n.no_storage && n.commuted_conv < 0) return;   // e.g. a ReLU in front of a depth-wise convolution that reads the summed inputs itself
        if (n.made_by_conv) return;  // addition (and ReLU) of a residual unit: the convolution's epilogue wrote this tensor
        // levels count inside a schedule unit; the members of a Sequential follow each other
        if (n.unit != level_unit_) {
            level_unit_ = n.unit;
            level_top_ = 0;
        }
        level_base_ = level_top_;
        int C, H, W;
        input_shape(n, C, H, W);
        const Json &cfg = *n.cfg;
        switch (n.type) {
            case NodeType::Conv:
                if (n.commuted_pool >= 0) emit_pool_behind_conv(n, index);
                else emit_conv(n, cfg, C, H, W, index);
                break;
            case NodeType::Pool:
                if (n.commuted_conv >= 0) emit_conv_before_pool(n, C, H, W, index);
                else emit_pool(n, cfg, C, H, W, index);
                break;
            case NodeType::Identity:
                if (!single_value(n)) emit_terms(n, index, ACT_NONE, false);
                break;
            case NodeType::Relu:
                if (!n.pre_relu_alias) emit_terms(n, index, ACT_RELU, false);
                break;
            case NodeType::Activation: emit_terms(n, index, act_code(cfg["act_type"].as_string()), false); break;
            case NodeType::Element: emit_terms(n, index, ACT_NONE, cfg["op_type"].as_string() == "mul"); break;
            default: break;
        }
    }

    void emit_terms(const PNode &n, int index, int act, bool multiply) {
        const ViewRef out = view_of(index);
        int offset = 0;
        if (n.combine_front >= 0) {
            const PNode &front = nodes_[n.combine_front];
            const bool product = front.type == NodeType::Element && (*front.cfg)["op_type"].as_string() == "mul";
            materialise_term(n, front.inputs[0], out, act, product);
            return;
        }
        for (const auto &term : n.inputs) {
            const int len = term[0].end - term[0].begin;
            bool in_place = false;
            if (term.size() == 1 && n.type == NodeType::Identity) {
                const PNode &p = nodes_[resolve_sequential(term[0].node)];
                in_place = p.fused_into == index && p.parent_begin == offset;
            }
            if (!in_place) materialise_term(n, term, out.window(offset, offset + len), act, multiply);
            offset += len;
        }
    }

    int add_plan_conv(const PNode &n, const ConvProblem &p) {
        PlanConv conv;
        conv.name = n.name;
        conv.problem = p;
        conv.weight_off = reserve((size_t)p.OC * p.K());
        conv.bias_off = reserve((size_t)p.OC);
        if (plan_.conv_index.count(n.name)) throw std::runtime_error("duplicate convolution name '" + n.name + "'");
        plan_.conv_index[n.name] = static_cast<int>(plan_.convs.size());
        plan_.convs.push_back(conv);
        return static_cast<int>(plan_.convs.size()) - 1;
    }

    void emit_conv(PNode &n, const Json &cfg, int C, int H, int W, int index) {
        (void)cfg;
        bool pre_relu = false;
        std::vector<ViewRef> sum_srcs;
        if (n.sum_front >= 0) {
            for (const Val &v : nodes_[n.sum_front].inputs[0]) sum_srcs.push_back(view_of(v.node).window(v.begin, v.end));
            pre_relu = n.sum_relu;
        }
        const ViewRef in = n.sum_front >= 0 ? sum_srcs[0] : input_view(n, C, H, W, &pre_relu);
        ConvProblem p = problem_of(n);
        p.pre_relu = pre_relu ? 1 : 0;
        OpKind kind;
        bool matrix_path = false;
        if (p.is_depthwise()) {
            kind = OpKind::ConvDepthwise;
        } else if ((p.groups > 1 && (p.ICg() < 4 || p.OCg() < 8)) || !conv_matrix_path_supported(p) ||
                   ((unsigned long long)(batch_ - 1) * in.bstride + in.image_floats()) * 4ull >= (1ull << 31)) {
            // thin groups, or an input view whose extent does not fit the matrix path's 31-bit byte offsets
            kind = OpKind::ConvDirect;
        } else {
            kind = OpKind::ConvMfma;
            matrix_path = true;
            // the kernel configuration depends on how many groups share the stage: chosen in finish()
        }
        const int conv = add_plan_conv(n, p);
        plan_.convs[conv].matrix_path = matrix_path;
        // K = 27: bound by the bytes of the output; from this size on the direct kernel with coalesced stores wins.  It is
        // not part of the fused stage kernel, so finish() keeps the matrix path when the stage turns out to have several groups.
        plan_.convs[conv].thin = matrix_path && conv_thin_applies(p) && planner_thin_conv_min_pixels() >= 0 &&
                                 p.Npix() >= planner_thin_conv_min_pixels() && p.Npix() * p.OC < (1LL << 31);
        PlanOp &op = push(kind, n);
        op.in = in;
        op.out = view_of(index);
        op.conv = conv;
        op.srcs = sum_srcs;
        const double k = sum_srcs.empty() ? 1.0 : (double)sum_srcs.size();
        op.flops = p.flops() + (k - 1.0) * (double)batch_ * C * H * W;
        op.bytes = 4.0 * (k * (double)batch_ * C * H * W + (double)p.OC * p.K() + p.OC + (double)batch_ * p.OC * p.OH * p.OW);
        if (n.residual_into >= 0) {
            const double out_elems = (double)batch_ * p.OC * p.OH * p.OW;
            const ViewRef other = view_of(n.residual_other.node).window(n.residual_other.begin, n.residual_other.end);
            if (matrix_path && !plan_.convs[conv].thin) {
                op.has_residual = true;
                op.residual = other;
                op.post_relu = n.residual_relu ? 1 : 0;
                op.flops += out_elems;
                op.bytes += 4.0 * out_elems;
            } else {
                // (an input view beyond the matrix path's offsets: the other kernels have no residual form, the sum follows
                // in place as a launch of its own)
                const ViewRef out = op.out;
                PlanOp &sum = push(OpKind::Nary, n);
                sum.srcs = {out, other};
                sum.out = out;
                sum.act = n.residual_relu ? ACT_RELU : ACT_NONE;
                sum.flops = out_elems;
                sum.bytes = 12.0 * out_elems;
                sum.level = level_base_ + 1;
                level_top_ = std::max(level_top_, sum.level + 1);
            }
        }
    }

    PoolProblem pool_problem_of(const PNode &n, int C, int H, int W) const {
        const Json &cfg = *n.cfg;
        const std::string pool_type = cfg["pool_type"].as_string();
        PoolProblem p;
        p.B = batch_; p.C = C; p.H = H; p.W = W;
        p.is_max = pool_type.find("max") != std::string::npos ? 1 : 0;
        if (pool_type.find("global") != std::string::npos) {
            p.KH = H; p.KW = W; p.sh = 1; p.sw = 1; p.ph = 0; p.pw = 0;
        } else {
            p.KH = cfg["kernel"][0].as_int(); p.KW = cfg["kernel"][1].as_int();
            p.sh = cfg["stride"][0].as_int(); p.sw = cfg["stride"][1].as_int();
            p.ph = cfg["padding"][0].as_int(); p.pw = cfg["padding"][1].as_int();
        }
        p.OH = n.H; p.OW = n.W;
        return p;
    }

    // the launch at the place of a commuted average pool (see find_commuting_pools): z = W * x into a temporary
    void emit_conv_before_pool(PNode &pool, int C, int H, int W, int index) {
        const PNode &c = nodes_[pool.commuted_conv];
        const ViewRef in = input_view(pool, C, H, W, nullptr);
        ConvProblem p = problem_of(c);
        p.act = ACT_NONE;
        const bool wide = ((unsigned long long)(batch_ - 1) * in.bstride + in.image_floats()) * 4ull >= (1ull << 31);
        const int conv = add_plan_conv(c, p);
        plan_.convs[conv].matrix_path = !wide;
        plan_.convs[conv].linear = true;
        plan_.convs[conv].zero_bias_off = reserve((size_t)p.OC);
        const ViewRef z = dense_temp(p.OC, H, W);
        commuted_z_[index] = z;
        PlanOp &op = push(wide ? OpKind::ConvDirect : OpKind::ConvMfma, pool);
        op.in = in;
        op.out = z;
        op.conv = conv;
        op.flops = p.flops();
        op.bytes = 4.0 * ((double)batch_ * C * H * W + (double)p.OC * p.K() + (double)batch_ * p.OC * H * W);
    }

    // the launch at the place of the convolution behind a commuted average pool: y = act(pool(z) + bias)
    void emit_pool_behind_conv(PNode &c, int index) {
        const PNode &pool = nodes_[c.commuted_pool];
        const ViewRef z = commuted_z_.at(c.commuted_pool);
        const PoolProblem p = pool_problem_of(pool, z.C, z.H, z.W);
        PlanOp &op = push(OpKind::Pool, c);
        op.in = z;
        op.out = view_of(index);
        op.pool = p;
        op.bias_conv = plan_.conv_index.at(c.name);
        op.act = act_code((*c.cfg)["act"].as_string());
        op.flops = (double)batch_ * z.C * p.OH * p.OW * (p.KH * p.KW + 1);
        op.bytes = 4.0 * ((double)batch_ * z.C * ((double)z.H * z.W + (double)p.OH * p.OW) + z.C);
    }

    void emit_pool(PNode &n, const Json &cfg, int C, int H, int W, int index) {
        const ViewRef in = input_view(n, C, H, W, nullptr);
        const bool global = cfg["pool_type"].as_string().find("global") != std::string::npos;
        const PoolProblem p = pool_problem_of(n, C, H, W);
        PlanOp &op = push(global ? OpKind::GlobalPool : OpKind::Pool, n);
        op.in = in;
        op.out = view_of(index);
        op.pool = p;
        op.flops = (double)batch_ * C * p.OH * p.OW * p.KH * p.KW;
        op.bytes = 4.0 * (double)batch_ * C * ((double)H * W + (double)p.OH * p.OW);
    }

    // ---- schedule -------------------------------------------------------------------------------------------------
    void assign_stages(const std::vector<std::vector<std::vector<std::string>>> &stage_names) {
        std::map<std::string, int> unit_of;
        for (size_t u = 0; u < units_.size(); u++) unit_of[units_[u]] = static_cast<int>(u);
        std::vector<std::vector<int>> ops_of_unit(units_.size());
        for (size_t i = 0; i < plan_.ops.size(); i++) ops_of_unit[plan_.ops[i].unit].push_back(static_cast<int>(i));
        // producers of every unit (as units), for the order check
        std::vector<std::set<int>> deps(units_.size());
        for (const PNode &n : nodes_) {
            if (n.unit < 0) continue;
            for (const auto &term : n.inputs)
                for (const Val &v : term) {
                    const int pu = nodes_[v.node].unit;
                    if (pu >= 0 && pu != n.unit) deps[n.unit].insert(pu);
                }
            if (n.residual_into >= 0) {   // the convolution's epilogue reads the other value of the addition
                const int pu = nodes_[n.residual_other.node].unit;
                if (pu >= 0 && pu != n.unit) deps[n.unit].insert(pu);
            }
        }
        std::vector<int> state(units_.size(), 0);   // 0 pending, 1 in the running stage, 2 finished
        std::vector<int> group_of(units_.size(), -1);
        for (size_t s = 0; s < stage_names.size(); s++) {
            const auto &groups = stage_names[s];
            if (groups.empty()) throw std::runtime_error("stage without groups");
            if (groups.size() > (size_t)kMaxGroups)
                throw std::runtime_error("The number of groups in stage " + std::to_string(s) + " exceeds the number of available streams " +
                                         std::to_string(kMaxGroups));
            std::vector<std::vector<int>> stage_ops(groups.size());
            for (size_t g = 0; g < groups.size(); g++) {
                for (const std::string &name : groups[g]) {
                    auto it = unit_of.find(name);
                    if (it == unit_of.end()) throw std::runtime_error("schedule names unknown operator '" + name + "'");
                    const int u = it->second;
                    if (state[u] != 0) throw std::runtime_error("operator '" + name + "' is scheduled twice");
                    for (int d : deps[u]) {
                        const bool ok = state[d] == 2 || (state[d] == 1 && group_of[d] == (int)g);
                        if (!ok)
                            throw std::runtime_error("schedule is not topological: '" + name + "' runs before or beside its input '" +
                                                     units_[d] + "'");
                    }
                    state[u] = 1;
                    group_of[u] = static_cast<int>(g);
                    for (int op : ops_of_unit[u]) {
                        plan_.ops[op].stage = static_cast<int>(s);
                        plan_.ops[op].group = static_cast<int>(g);
                        stage_ops[g].push_back(op);
                    }
                }
            }
            for (int &st : state)
                if (st == 1) st = 2;
            plan_.stages.push_back(stage_ops);
        }
        for (size_t u = 0; u < units_.size(); u++)
            if (state[u] == 0) throw std::runtime_error("operator '" + units_[u] + "' is missing from the schedule");
        plan_.output_single_group = stage_names.back().size() == 1;
    }

    void finish() {
        for (size_t i = 0; i < nodes_.size(); i++) {
            const PNode &n = nodes_[i];
            if (n.pre_relu_alias || n.no_storage || n.residual_into >= 0) continue;   // never materialised
            plan_.tensors[n.name] = view_of(static_cast<int>(i));
        }
        plan_.input = view_of(0);
        // the result is the last operator of the last stage's last group
        const auto &last_stage_units = unit_result_;
        int out_node = last_stage_units.back();
        plan_.output = view_of(out_node);
        plan_.output_name = nodes_[out_node].name;
        std::vector<int> share(plan_.convs.size(), 1);
        // a convolution shares the device with the operators at the same position of the other groups of its stage
        // (the fused executor runs position after position); in a multi-group stage it counts at least two, because
        // it must be able to run inside a fused launch even when it is the only operator left at its position
        for (const auto &stage : plan_.stages)
            for (const auto &group : stage)
                for (size_t pos = 0; pos < group.size(); pos++) {
                    const PlanOp &op = plan_.ops[group[pos]];
                    if (op.conv < 0) continue;
                    int busy = 0;
                    for (const auto &other : stage) busy += other.size() > pos ? 1 : 0;
                    share[op.conv] = stage.size() > 1 ? std::max(2, busy) : 1;
                }
        for (PlanOp &op : plan_.ops) {
            if (op.conv < 0 || !plan_.convs[op.conv].thin) continue;
            PlanConv &conv = plan_.convs[op.conv];
            if (plan_.stages[op.stage].size() == 1) {
                conv.matrix_path = false;
                op.kind = OpKind::ConvDirect;
            } else {
                conv.thin = false;
            }
        }
        for (size_t i = 0; i < plan_.convs.size(); i++) {
            PlanConv &conv = plan_.convs[i];
            if (!conv.matrix_path) continue;
            conv.launch = chooser_(conv.problem, share[i]);
            conv.packed_off = reserve(conv_packed_floats(conv.problem, conv.launch));
            conv.ws_floats = conv_workspace_floats(conv.problem, conv.launch);
            if (conv.ws_floats > 0) conv.ws_off = reserve_region(conv.ws_floats);
            conv.ctr_count = conv_counter_count(conv.problem, conv.launch);
            if (conv.ctr_count > 0) conv.ctr_off = reserve(conv.ctr_count);
        }
        place_regions();
    }

    int batch_;
    int level_unit_ = -2, level_base_ = 0, level_top_ = 0;   // PlanOp::level of the operations being emitted
    const LaunchChooser &chooser_;
    Plan plan_;
    std::vector<PNode> nodes_;
    std::map<std::string, int> by_name_;
    std::vector<std::string> units_;
    std::vector<int> unit_result_;
    struct Slot {
        int stage = -1, group = -1, pos = -1;
    };
    std::vector<Slot> slots_;
    std::vector<int> groups_in_stage_;
    struct SeqRange { int first, second; };
    std::vector<SeqRange> sequentials_;
    std::vector<Region> regions_;   // ascending virtual offsets
    size_t region_floats_ = 0;
    std::map<int, ViewRef> commuted_z_;   // commuted pool node -> the temporary between the convolution and the pool
};

void json_escape(std::ostringstream &os, const std::string &s) {
    os << '"';
    for (char c : s) {
        if (c == '"' || c == '\\') os << '\\' << c;
        else if ((unsigned char)c < 0x20) os << ' ';
        else os << c;
    }
    os << '"';
}

}  // namespace

namespace {
bool g_arena_reuse = true;
long long g_thin_conv_min_pixels = 1LL << 18;
int g_host_split_k = 0;
bool g_commute_pool_conv = true;
}

bool set_planner_option(const std::string &key, const std::string &value) {
    if (key == "arena_reuse") {
        g_arena_reuse = !(value == "0" || value == "false" || value == "off" || value.empty());
        return true;
    }
    if (key == "commute_pool_conv") {
        g_commute_pool_conv = !(value == "0" || value == "false" || value == "off" || value.empty());
        return true;
    }
    if (key == "thin_conv_min_pixels") {
        g_thin_conv_min_pixels = atoll(value.c_str());
        return true;
    }
    if (key == "host_plan_split_k") {   // K slices of every matrix-path convolution in plans made without a device (0: the model's choice)
        const int v = atoi(value.c_str());
        if (v < 0 || v > 64) throw std::runtime_error("option host_plan_split_k: expected 0..64");
        g_host_split_k = v;
        return true;
    }
    return false;
}

bool planner_arena_reuse() { return g_arena_reuse; }
long long planner_thin_conv_min_pixels() { return g_thin_conv_min_pixels; }
int planner_host_split_k() { return g_host_split_k; }
bool planner_commute_pool_conv() { return g_commute_pool_conv; }

Plan build_plan(PlanMode mode, const Json &doc, const Json *extra, int batch, const LaunchChooser &chooser) {
    Planner planner(batch, chooser);
    return planner.run(mode, doc, extra);
}

std::string describe_plan(const Plan &plan) {
    std::ostringstream os;
    os << '[';
    for (size_t i = 0; i < plan.ops.size(); i++) {
        const PlanOp &op = plan.ops[i];
        if (i) os << ',';
        os << "{\"index\":" << i << ",\"node\":";
        json_escape(os, op.node);
        os << ",\"unit\":";
        json_escape(os, plan.unit_names[op.unit]);
        os << ",\"kind\":\"" << op_kind_name(op.kind) << "\",\"stage\":" << op.stage << ",\"group\":" << op.group;
        os << ",\"flops\":" << op.flops << ",\"bytes\":" << op.bytes;
        os << ",\"out\":[" << op.out.C << ',' << op.out.H << ',' << op.out.W << "],\"out_bstride\":" << op.out.bstride;
        if (op.conv >= 0) {
            const PlanConv &c = plan.convs[op.conv];
            const ConvProblem &p = c.problem;
            os << ",\"conv\":{\"ic\":" << p.IC << ",\"h\":" << p.H << ",\"w\":" << p.W << ",\"oc\":" << p.OC << ",\"kh\":" << p.KH
               << ",\"kw\":" << p.KW << ",\"sh\":" << p.sh << ",\"sw\":" << p.sw << ",\"ph\":" << p.ph << ",\"pw\":" << p.pw
               << ",\"groups\":" << p.groups << ",\"act\":" << p.act << ",\"pre_relu\":" << p.pre_relu << "}";
            if (op.kind == OpKind::ConvDirect) os << ",\"thin\":" << (c.thin ? "true" : "false");
            if (c.matrix_path) {
                os << ",\"variant\":\"" << conv_variant(c.launch.variant).name << "\",\"split_k\":" << c.launch.split_k
                   << ",\"fusable\":" << (conv_variant(c.launch.variant).fusable() ? "true" : "false");
            }
        }
        if (op.kind == OpKind::Nary) os << ",\"inputs\":" << op.srcs.size() << ",\"accumulate\":" << op.accumulate;
        if (op.kind == OpKind::ConvDepthwise) os << ",\"inputs\":" << (op.srcs.empty() ? 1 : op.srcs.size());
        if (op.kind == OpKind::Nary || op.kind == OpKind::Unary) os << ",\"act\":" << op.act;
        if (op.bias_conv >= 0) os << ",\"adds_bias_of\":\"" << plan.convs[op.bias_conv].name << "\",\"act\":" << op.act;
        if (op.conv >= 0 && plan.convs[op.conv].linear) os << ",\"linear\":true";
        if (op.has_residual) os << ",\"residual\":true,\"post_relu\":" << op.post_relu;
        os << ",\"level\":" << op.level;
        // arena extents in floats, one [begin, end) per image: what the operation writes and what it reads
        auto ranges = [&](const char *key, const std::vector<ViewRef> &views) {
            os << ",\"" << key << "\":[";
            bool first_range = true;
            for (const ViewRef &v : views)
                for (int n = 0; n < plan.batch; n++) {
                    const size_t begin = v.offset + (size_t)n * (size_t)v.bstride;
                    os << (first_range ? "" : ",") << '[' << begin << ',' << begin + v.image_floats() << ']';
                    first_range = false;
                }
            os << ']';
        };
        std::vector<ViewRef> reads = op.srcs;
        if (op.kind != OpKind::Nary && op.srcs.empty()) reads.push_back(op.in);
        if (op.kind == OpKind::Nary && op.accumulate) reads.push_back(op.out);
        if (op.has_residual) reads.push_back(op.residual);
        ranges("writes", {op.out});
        ranges("reads", reads);
        // a split-K convolution first writes, then reads its partial tiles: a region that shares addresses with other tensors
        // like any other
        if (op.conv >= 0 && plan.convs[op.conv].ws_floats > 0) {
            const PlanConv &c = plan.convs[op.conv];
            os << ",\"scratch\":[[" << c.ws_off << ',' << c.ws_off + c.ws_floats << "]]";
        }
        os << '}';
    }
    os << ']';
    return os.str();
}

}  // namespace ios
