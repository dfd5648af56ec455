#include "fusion.h"

#include <cstdio>
#include <cstring>
#include <map>
#include <queue>
#include <sstream>
#include <stack>

#include "../runtime/log.h"

namespace chainer_compiler {

namespace {

// A candidate that can be reached from the set through a node outside the set would close a
// cycle through the fused node: walk down from every outside user and drop what is met.
void RejectCyclicNodes(std::set<Node*>* cands) {
    std::stack<Node*> q;
    for (Node* node : *cands)
        for (Value* output : node->outputs())
            for (Node* n : output->users())
                if (!cands->count(n)) q.push(n);
    std::set<Node*> rejected, seen;
    while (!q.empty()) {
        Node* node = q.top();
        q.pop();
        if (!seen.insert(node).second) continue;
        if (cands->count(node)) rejected.insert(node);
        for (Value* output : node->outputs())
            for (Node* n : output->users()) q.push(n);
    }
    for (Node* node : rejected) cands->erase(node);
}

void RejectUnusedConstants(std::set<Node*>* cands) {
    std::set<Node*> rejected;
    for (Node* node : *cands) {
        if (node->op_type() != "Constant") continue;
        bool used = false;
        for (Node* user : node->output(0)->users())
            if (cands->count(user)) used = true;
        if (!used) rejected.insert(node);
    }
    for (Node* node : rejected) cands->erase(node);
}

std::string MakeValueName(const char* prefix, int index, const std::string& name) {
    CHECK_LT(index, 1000);
    char buf[16];
    snprintf(buf, sizeof(buf), "%03d", index);
    return std::string(prefix) + buf + "_" + name;
}

bool IsOneElementFloatConstant(const Node& node) {
    if (node.op_type() != "Constant") return false;
    std::unique_ptr<Tensor> t = node.tensor_value();
    return t && DtypeIsFloat(t->dtype()) && t->NumElements() == 1;
}

bool OperandsAreFloat(const Node& node) {
    for (Value* v : node.inputs()) {
        const CDtype dt = v->type().dtype;
        if (!DtypeIsFloat(dt) && dt != kUnknown) return false;
    }
    return true;
}

// the one-element constant behind a value (initializer or Constant node), or null
std::unique_ptr<Tensor> OneElementConstant(const Value* v) {
    std::unique_ptr<Tensor> t;
    if (v->initializer()) t = std::make_unique<Tensor>(*v->initializer());
    else if (v->producer() && v->producer()->op_type() == "Constant") t = v->producer()->tensor_value();
    if (t && t->NumElements() == 1) return t;
    return nullptr;
}

}  // namespace

void CreateFusionGroup(Graph* graph, const std::set<Node*>& nodes, const std::string& fusion_type, int fusion_group_id,
                       bool can_fuse_initializers) {
    std::vector<Value*> inputs, outputs, temps;
    ClassifyValues(std::vector<Node*>(nodes.begin(), nodes.end()), &inputs, &outputs, &temps);
    if (inputs.empty() || outputs.empty()) return;

    GraphBuilder gb(graph, "Fusion" + std::to_string(fusion_group_id), outputs.front());
    auto replace_value = [&nodes](Value* value, Value* new_value) {
        if (Node* producer = value->producer())
            if (nodes.count(producer)) producer->ReplaceOutput(value, new_value);
        const std::vector<Node*> users(value->users());  // a copy: the list changes underneath
        for (Node* user : users)
            if (nodes.count(user)) user->ReplaceInput(value, new_value);
    };

    std::unique_ptr<Graph> subgraph(new Graph("Fusion_" + std::to_string(fusion_group_id)));
    std::vector<Value*> subgraph_inputs;
    for (size_t i = 0; i < inputs.size(); ++i) {
        Value* value = inputs[i];
        const std::string new_name = MakeValueName("fi", static_cast<int>(i), value->name());
        Value* new_value = subgraph->AddInputValue(new_name, value->type());
        replace_value(value, new_value);
        if (can_fuse_initializers && value->initializer()) {
            new_value->ResetInitializer(std::make_unique<Tensor>(*value->initializer()));
        } else {
            subgraph_inputs.push_back(value);
        }
    }
    for (size_t i = 0; i < outputs.size(); ++i) {
        Value* value = outputs[i];
        Value* new_value = subgraph->AddOutputValue(MakeValueName("fo", static_cast<int>(i), value->name()), value->type());
        replace_value(value, new_value);
    }
    Node* fused = gb.MOp("ChainerFusionGroup", subgraph_inputs, outputs);
    graph->MigrateNodes(std::vector<Node*>(nodes.begin(), nodes.end()), temps, subgraph.get());
    fused->set_subgraph(std::move(subgraph));
    fused->set_fusion_type(fusion_type);
    fused->set_chainer_fusion_group(fusion_group_id);
}

int FuseAllConnectedNodes(const char* name, Graph* graph, int min_fuse_ops, bool can_fuse_initializers,
                          const std::function<bool(const Node&)>& is_fusable,
                          const std::function<bool(const Node& producer, const Node& user)>& can_cross) {
    int num_fusion_groups = 0;
    const std::vector<Node*> all_nodes(graph->GetLiveNodes());
    for (Node* base_node : all_nodes) {
        if (base_node->detached() || base_node->chainer_fusion_group()) continue;
        if (!is_fusable(*base_node)) continue;
        std::set<Node*> cands;
        std::stack<Node*> q;
        q.push(base_node);
        while (!q.empty()) {
            Node* node = q.top();
            q.pop();
            if (node->chainer_fusion_group()) continue;
            if (!cands.insert(node).second) continue;
            for (Value* value : node->inputs()) {
                Node* next = value->producer();
                if (next && !next->chainer_fusion_group() && is_fusable(*next) && (!can_cross || can_cross(*next, *node))) q.push(next);
            }
            for (Value* value : node->outputs())
                for (Node* next : value->users())
                    if (!next->chainer_fusion_group() && is_fusable(*next) && (!can_cross || can_cross(*node, *next))) q.push(next);
        }
        RejectCyclicNodes(&cands);
        RejectUnusedConstants(&cands);
        int num_calculation = 0;
        for (Node* node : cands)
            if (!node->IsZeroCost()) ++num_calculation;
        if (num_calculation < min_fuse_ops) continue;
        ++num_fusion_groups;
        for (Node* node : cands) node->set_chainer_fusion_group(num_fusion_groups);
        CreateFusionGroup(graph, cands, name, num_fusion_groups, can_fuse_initializers);
    }
    return num_fusion_groups;
}

int FuseElementwiseOperations(Graph* graph) {
    static const std::set<std::string> fusable_ops = {"Identity", "Add", "Sub", "Mul", "Tanh", "Sigmoid", "Exp"};
    auto is_fusable = [](const Node& node) {
        if (node.op_type() == "Constant") return IsOneElementFloatConstant(node);
        return fusable_ops.count(node.op_type()) > 0 && OperandsAreFloat(node);
    };
    return FuseAllConnectedNodes("nvrtc", graph, 2, false, is_fusable);
}

int FuseHipOperations(Graph* graph) {
    static const std::set<std::string> float_ops = {"Identity", "Add", "Sub", "Mul", "Div", "Neg", "Tanh", "Sigmoid", "Exp", "Relu", "Abs", "Floor", "Round"};
    auto constant_operands = [](const Node& node, size_t first) {
        for (size_t i = first; i < node.inputs().size(); ++i) {
            if (node.input(i)->IsNull()) continue;
            if (!OneElementConstant(node.input(i))) return false;
        }
        return true;
    };
    auto is_fusable = [&](const Node& node) {
        const std::string& op = node.op_type();
        if (op == "Constant") return IsOneElementFloatConstant(node);
        if (float_ops.count(op)) return OperandsAreFloat(node);
        if (op == "Max" || op == "Min") return node.inputs().size() == 2 && OperandsAreFloat(node);
        if (op == "Clip") {
            // bounds as attributes (opset < 11) or as constant operands
            const CDtype dt = node.input(0)->type().dtype;
            return (DtypeIsFloat(dt) || dt == kUnknown) && constant_operands(node, 1);
        }
        if (op == "QuantizeLinear") {
            const CDtype dt = node.input(0)->type().dtype;
            return (DtypeIsFloat(dt) || dt == kUnknown) && node.inputs().size() >= 2 && constant_operands(node, 1);
        }
        if (op == "DequantizeLinear") {
            // Only where it opens an element-wise computation.  In front of anything else (a pool, a
            // float convolution) it stays an instruction of its own: the runtime pairs
            // DequantizeLinear -> pool -> QuantizeLinear into its quantized pool kernels, and a
            // group that swallowed the DequantizeLinear would leave a float pool behind.
            if (!(node.inputs().size() >= 2 && constant_operands(node, 1))) return false;
            for (Node* user : node.output(0)->users()) {
                const std::string& u = user->op_type();
                if (!float_ops.count(u) && u != "Max" && u != "Min" && u != "Clip" && u != "QuantizeLinear") return false;
            }
            return true;
        }
        return false;
    };
    // A QuantizeLinear closes an element-wise computation and a DequantizeLinear opens the next one:
    // the 8-bit tensor between them is an activation of the network (other nodes read it, the
    // runtime keeps it channels-last), so groups do not grow across that edge.
    // One kernel writes every output of a group in one shape (the broadcast of its operands,
    // runtime/ops/nvrtc.cc:100-104), so two nodes whose results are known to differ in shape (a 0-d
    // scale and the [OC] vector it is multiplied into) do not share a group.
    auto can_cross = [](const Node& producer, const Node& user) {
        if (producer.op_type() == "QuantizeLinear" && user.op_type() == "DequantizeLinear") return false;
        if (producer.op_type() == "Constant") return true;  // read in place by the kernel, no output of its own
        const Type& a = producer.output(0)->type();
        const Type& b = user.output(0)->type();
        if (a.has_dims && b.has_dims && a.dims != b.dims) return false;
        return true;
    };
    return FuseAllConnectedNodes("hip", graph, 2, false, is_fusable, can_cross);
}

// ---- program text -------------------------------------------------------------------------------

namespace {

std::string CleanseIdent(const std::string& s) {
    std::string o = "v_";
    for (char c : s) o += (isalnum(static_cast<unsigned char>(c)) ? c : '_');
    return o;
}

std::string FloatBits(double v) {
    const float f = static_cast<float>(v);
    uint32_t bits;
    memcpy(&bits, &f, 4);
    char buf[16];
    snprintf(buf, sizeof(buf), "0x%08x", bits);
    return buf;
}

const char* PortDtype(CDtype dt) {
    switch (dt) {
        case kUInt8: return "uint8";
        case kInt8: return "int8";
        case kFloat32: case kUnknown: return "float32";
        default: CHECK(false) << "the hip fusion back-end has no element type " << DtypeName(dt);
    }
    return "";
}

}  // namespace

std::string BuildHipProgram(const Node& group, std::vector<int>* used_inputs) {
    CHECK(group.subgraph()) << group.ToString() << " is not a fusion group";
    const Graph& body = *group.subgraph();
    CHECK_EQ(group.inputs().size(), body.input_values().size()) << "initializers are not fused into hip groups";
    std::ostringstream os;
    // dtypes: what the graph says; a value nobody typed is float32, as in BuildNvrtcProgram
    std::map<const Value*, CDtype> dtype;
    // A group input that only parametrizes a QuantizeLinear / DequantizeLinear / Clip (scale, zero
    // point, bound) is a constant of the outer graph: it is written into the statement and is no
    // operand of the kernel.
    std::map<const Value*, std::unique_ptr<Tensor>> constants;
    std::set<const Value*> data_inputs, absent;
    for (Node* node : body.GetLiveNodes()) {
        const std::string& op = node->op_type();
        const size_t first_param = (op == "QuantizeLinear" || op == "DequantizeLinear" || op == "Clip") ? 1 : node->inputs().size();
        for (size_t i = 0; i < node->inputs().size() && i < first_param; ++i) data_inputs.insert(node->input(i));
    }
    used_inputs->clear();
    os << "chxhip-fusion 1\nin";
    for (size_t i = 0; i < body.input_values().size(); ++i) {
        Value* v = body.input_values()[i];
        if (!data_inputs.count(v)) {
            if (group.input(static_cast<int>(i))->IsNull()) {  // an absent bound of a Clip
                absent.insert(v);
                continue;
            }
            constants[v] = OneElementConstant(group.input(static_cast<int>(i)));
            CHECK(constants[v]) << "parameter '" << group.input(static_cast<int>(i))->name() << "' of the group is not a one-element constant";
            continue;
        }
        used_inputs->push_back(static_cast<int>(i));
        dtype[v] = v->type().dtype == kUnknown ? kFloat32 : v->type().dtype;
        os << " " << CleanseIdent(v->name()) << ":" << PortDtype(dtype[v]);
    }
    os << "\n";

    std::map<Node*, int> input_counts;
    for (Node* node : body.GetLiveNodes()) input_counts[node] = node->GetNumActualInputs();
    std::queue<Value*> q;
    for (Value* v : body.input_values()) q.push(v);
    // one-element constants become literals; the parameters of Q/DQ/Clip are read where they are used
    for (Node* node : body.GetLiveNodes()) {
        if (node->op_type() != "Constant") continue;
        std::unique_ptr<Tensor> t = node->tensor_value();
        CHECK(t && t->NumElements() == 1) << node->ToString();
        os << CleanseIdent(node->output(0)->name()) << " = Const " << FloatBits(t->GetAsDouble(0)) << "\n";
        dtype[node->output(0)] = kFloat32;
        constants[node->output(0)] = std::move(t);
        q.push(node->output(0));
    }
    auto constant_of = [&](const Value* v) -> const Tensor* {
        auto it = constants.find(v);
        CHECK(it != constants.end()) << "'" << v->name() << "' is not a constant of the group";
        return it->second.get();
    };
    auto emit = [&](Node* node) {
        std::vector<std::string> ins;
        for (Value* v : node->inputs()) ins.push_back(v->IsNull() ? "" : CleanseIdent(v->name()));
        const std::string out = CleanseIdent(node->output(0)->name());
        const std::string& op = node->op_type();
        CDtype out_dtype = kFloat32;
        if (op == "Identity" || op == "Neg" || op == "Tanh" || op == "Sigmoid" || op == "Exp" || op == "Relu" || op == "Abs" ||
            op == "Floor" || op == "Round") {
            os << out << " = " << op << " " << ins[0] << "\n";
        } else if (op == "Add" || op == "Sub" || op == "Mul" || op == "Div" || op == "Max" || op == "Min") {
            CHECK_EQ(2UL, ins.size()) << node->ToString();
            os << out << " = " << op << " " << ins[0] << " " << ins[1] << "\n";
        } else if (op == "Clip") {
            double lo = node->GetFloat("min", -3.4028234663852886e38f), hi = node->GetFloat("max", 3.4028234663852886e38f);
            auto given = [&](size_t i) { return node->inputs().size() > i && !node->input(i)->IsNull() && !absent.count(node->input(i)); };
            if (given(1)) lo = constant_of(node->input(1))->GetAsDouble(0);
            if (given(2)) hi = constant_of(node->input(2))->GetAsDouble(0);
            os << out << " = Clip " << ins[0] << " " << FloatBits(lo) << " " << FloatBits(hi) << "\n";
        } else if (op == "QuantizeLinear" || op == "DequantizeLinear") {
            const double scale = constant_of(node->input(1))->GetAsDouble(0);
            int64_t zp = 0;
            CDtype zdt = kUInt8;
            if (node->inputs().size() > 2 && !node->input(2)->IsNull()) {
                zp = static_cast<int64_t>(constant_of(node->input(2))->GetAsDouble(0));
                zdt = constant_of(node->input(2))->dtype();
            }
            if (op == "QuantizeLinear") {
                os << out << " = QuantizeLinear " << ins[0] << " " << FloatBits(scale) << " " << zp << " " << PortDtype(zdt) << "\n";
                out_dtype = zdt;
            } else {
                os << out << " = DequantizeLinear " << ins[0] << " " << FloatBits(scale) << " " << zp << "\n";
            }
        } else {
            CHECK(false) << "cannot build a hip program for " << node->ToString();
        }
        dtype[node->output(0)] = out_dtype;
    };
    // Q/DQ/Clip parameters are constants of the group that feed no statement of their own: they must
    // not hold their reader back, and integer constants never become Const statements
    while (!q.empty()) {
        Value* value = q.front();
        q.pop();
        for (Node* node : value->users()) {
            auto found = input_counts.find(node);
            if (found == input_counts.end()) continue;
            if (--found->second != 0) continue;
            emit(node);
            for (Value* o : node->outputs()) q.push(o);
        }
    }
    os << "out";
    for (Value* v : body.output_values()) {
        CHECK(dtype.count(v)) << "output '" << v->name() << "' of the group was never computed";
        os << " " << CleanseIdent(v->name()) << ":" << PortDtype(dtype[v]);
    }
    os << "\n";
    return os.str();
}

}  // namespace chainer_compiler
