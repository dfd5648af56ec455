#include "graph.h"

#include <algorithm>
#include <climits>
#include <cstring>
#include <queue>
#include <sstream>

#include "../runtime/log.h"

namespace chainer_compiler {

CDtype DtypeFromOnnx(int d) {
    switch (d) {
        case kOnnxFloat: return kFloat32;
        case kOnnxDouble: return kFloat64;
        case kOnnxUInt8: return kUInt8;
        case kOnnxInt8: return kInt8;
        case kOnnxInt32: return kInt32;
        case kOnnxInt64: return kInt64;
        case kOnnxBool: return kBool;
        default: return kUnknown;
    }
}

int DtypeToOnnx(CDtype d) {
    switch (d) {
        case kFloat32: return kOnnxFloat;
        case kFloat64: return kOnnxDouble;
        case kUInt8: return kOnnxUInt8;
        case kInt8: return kOnnxInt8;
        case kInt32: return kOnnxInt32;
        case kInt64: return kOnnxInt64;
        case kBool: return kOnnxBool;
        default: return 0;
    }
}

int DtypeSize(CDtype d) {
    switch (d) {
        case kBool: case kInt8: case kUInt8: return 1;
        case kInt16: case kFloat16: return 2;
        case kInt32: case kFloat32: return 4;
        case kInt64: case kFloat64: return 8;
        default: return 0;
    }
}

bool DtypeIsFloat(CDtype d) {
    return d == kFloat16 || d == kFloat32 || d == kFloat64;
}

const char* DtypeName(CDtype d) {
    static const char* names[] = {"unknown", "bool", "int8", "int16", "int32", "int64", "uint8", "float16", "float32", "float64"};
    return names[d];
}

// ---- Tensor ------------------------------------------------------------------------------------

Tensor::Tensor(std::string name, CDtype dtype, std::vector<int64_t> dims, std::string raw)
    : name_(std::move(name)), dtype_(dtype), dims_(std::move(dims)), raw_(std::move(raw)) {
    CHECK_EQ(static_cast<int64_t>(raw_.size()), NumElements() * DtypeSize(dtype_)) << "tensor '" << name_ << "'";
}

Tensor Tensor::FromOnnx(const OnnxTensor& t) {
    const CDtype dt = DtypeFromOnnx(t.dtype);
    CHECK(dt != kUnknown) << "tensor '" << t.name << "': unsupported element type " << t.dtype;
    return Tensor(t.name, dt, t.dims, t.raw);
}

OnnxTensor Tensor::ToOnnx() const {
    OnnxTensor t;
    t.name = name_;
    t.dtype = DtypeToOnnx(dtype_);
    CHECK(t.dtype) << "tensor '" << name_ << "' has no ONNX element type";
    t.dims = dims_;
    t.raw = raw_;
    return t;
}

int64_t Tensor::NumElements() const {
    int64_t n = 1;
    for (int64_t d : dims_) n *= d;
    return n;
}

double Tensor::GetAsDouble(int64_t i) const {
    CHECK(i >= 0 && i < NumElements());
    const char* p = raw_.data() + i * DtypeSize(dtype_);
    switch (dtype_) {
        case kFloat32: { float v; memcpy(&v, p, 4); return v; }
        case kFloat64: { double v; memcpy(&v, p, 8); return v; }
        case kInt8: return *reinterpret_cast<const int8_t*>(p);
        case kUInt8: case kBool: return *reinterpret_cast<const uint8_t*>(p);
        case kInt32: { int32_t v; memcpy(&v, p, 4); return v; }
        case kInt64: { int64_t v; memcpy(&v, p, 8); return static_cast<double>(v); }
        default: CHECK(false) << "tensor '" << name_ << "': cannot read " << DtypeName(dtype_);
    }
    return 0;
}

std::vector<float> Tensor::AsFloats() const {
    std::vector<float> out(NumElements());
    for (int64_t i = 0; i < NumElements(); ++i) out[i] = static_cast<float>(GetAsDouble(i));
    return out;
}

// ---- Value / Node ------------------------------------------------------------------------------

const Tensor* Value::GetConstTensor() const {
    if (initializer_) return initializer_.get();
    return nullptr;
}

Node::Node(std::string name, std::string op_type, std::vector<Value*> inputs, std::vector<Value*> outputs)
    : name_(std::move(name)), op_type_(std::move(op_type)), inputs_(std::move(inputs)), outputs_(std::move(outputs)) {
    for (Value* v : inputs_) v->users_.push_back(this);
    for (Value* v : outputs_) {
        CHECK(v->IsNull() || !v->producer_) << "value '" << v->name() << "' already has a producer";
        if (!v->IsNull()) v->producer_ = this;
    }
}

void Node::ReplaceInput(Value* from, Value* to) {
    bool found = false;
    for (Value*& v : inputs_)
        if (v == from) {
            v = to;
            found = true;
            to->users_.push_back(this);
        }
    CHECK(found) << "'" << from->name() << "' is not an input of " << ToString();
    from->users_.erase(std::remove(from->users_.begin(), from->users_.end(), this), from->users_.end());
}

void Node::ReplaceOutput(Value* from, Value* to) {
    bool found = false;
    for (Value*& v : outputs_)
        if (v == from) {
            v = to;
            found = true;
        }
    CHECK(found) << "'" << from->name() << "' is not an output of " << ToString();
    from->producer_ = nullptr;
    to->producer_ = this;
}

int Node::GetNumActualInputs() const {
    int n = 0;
    for (Value* v : inputs_) n += !v->IsNull();
    return n;
}

const OnnxAttr* Node::FindAttr(const std::string& name) const {
    for (const OnnxAttr& a : attrs_)
        if (a.name == name) return &a;
    return nullptr;
}

int64_t Node::GetInt(const std::string& name, int64_t def) const {
    const OnnxAttr* a = FindAttr(name);
    return a ? a->i : def;
}

float Node::GetFloat(const std::string& name, float def) const {
    const OnnxAttr* a = FindAttr(name);
    return a ? a->f : def;
}

std::string Node::GetString(const std::string& name, const std::string& def) const {
    const OnnxAttr* a = FindAttr(name);
    return a ? a->s : def;
}

std::vector<int64_t> Node::GetInts(const std::string& name) const {
    const OnnxAttr* a = FindAttr(name);
    return a ? a->ints : std::vector<int64_t>();
}

namespace {
OnnxAttr* AttrSlot(std::vector<OnnxAttr>* attrs, const std::string& name) {
    for (OnnxAttr& a : *attrs)
        if (a.name == name) {
            a = OnnxAttr();
            a.name = name;
            return &a;
        }
    attrs->emplace_back();
    attrs->back().name = name;
    return &attrs->back();
}
}  // namespace

void Node::SetInt(const std::string& name, int64_t v) {
    OnnxAttr* a = AttrSlot(&attrs_, name);
    a->type = OnnxAttr::kInt;
    a->i = v;
}

void Node::SetInts(const std::string& name, const std::vector<int64_t>& v) {
    OnnxAttr* a = AttrSlot(&attrs_, name);
    a->type = OnnxAttr::kInts;
    a->ints = v;
}

void Node::SetString(const std::string& name, const std::string& v) {
    OnnxAttr* a = AttrSlot(&attrs_, name);
    a->type = OnnxAttr::kString;
    a->s = v;
}

void Node::SetTensor(const std::string& name, const Tensor& t) {
    OnnxAttr* a = AttrSlot(&attrs_, name);
    a->type = OnnxAttr::kTensor;
    a->t = t.ToOnnx();
}

void Node::CopyAttrsFrom(const Node& other, const std::vector<std::string>& names) {
    for (const std::string& n : names)
        if (const OnnxAttr* a = other.FindAttr(n)) *AttrSlot(&attrs_, n) = *a;
}

std::unique_ptr<Tensor> Node::tensor_value() const {
    const OnnxAttr* a = FindAttr("value");
    if (!a || a->type != OnnxAttr::kTensor) return nullptr;
    return std::make_unique<Tensor>(Tensor::FromOnnx(a->t));
}

void Node::set_subgraph(std::unique_ptr<Graph> g) {
    subgraph_ = std::move(g);
}

std::string Node::ToString() const {
    std::ostringstream oss;
    oss << op_type_ << "(";
    for (size_t i = 0; i < inputs_.size(); ++i) oss << (i ? ", " : "") << inputs_[i]->name();
    oss << ") -> (";
    for (size_t i = 0; i < outputs_.size(); ++i) oss << (i ? ", " : "") << outputs_[i]->name();
    oss << ")";
    return oss.str();
}

// ---- Graph -------------------------------------------------------------------------------------

Graph::~Graph() = default;

Value* Graph::AddValue(const std::string& name, const Type& type, Value::Kind kind) {
    all_values_.emplace_back(new Value(name, type, kind));
    Value* v = all_values_.back().get();
    if (kind == Value::kInput) input_values_.push_back(v);
    else if (kind == Value::kOutput) output_values_.push_back(v);
    else if (kind == Value::kTemp) temp_values_.push_back(v);
    return v;
}

Node* Graph::AddNode(const std::string& op_type, const std::vector<Value*>& inputs, const std::vector<Value*>& outputs,
                     const std::string& base_name) {
    all_nodes_.emplace_back(new Node(GenSym(base_name.empty() ? op_type : base_name), op_type, inputs, outputs));
    nodes_.push_back(all_nodes_.back().get());
    return nodes_.back();
}

void Graph::DetachNode(Node* node) {
    for (Value* v : node->inputs_) v->users_.erase(std::remove(v->users_.begin(), v->users_.end(), node), v->users_.end());
    for (Value* v : node->outputs_)
        if (v->producer_ == node) v->producer_ = nullptr;
    node->inputs_.clear();
    node->outputs_.clear();
    node->detached_ = true;
}

std::vector<Node*> Graph::GetLiveNodes() const {
    std::vector<Node*> out;
    for (Node* n : nodes_)
        if (!n->detached()) out.push_back(n);
    return out;
}

std::vector<Node*> Graph::GetTopologicallySortedNodes() const {
    // Kahn's algorithm over the live nodes; ties keep creation order
    const std::vector<Node*> live = GetLiveNodes();
    std::map<Node*, int> pending;
    for (Node* n : live) {
        int c = 0;
        for (Value* v : n->inputs())
            if (v->producer() && !v->producer()->detached()) ++c;
        pending[n] = c;
    }
    std::vector<Node*> out;
    std::vector<bool> done(live.size(), false);
    while (out.size() < live.size()) {
        bool progress = false;
        for (size_t i = 0; i < live.size(); ++i) {
            if (done[i] || pending[live[i]] != 0) continue;
            done[i] = true;
            progress = true;
            out.push_back(live[i]);
            for (Value* o : live[i]->outputs())
                for (Node* u : o->users())
                    if (pending.count(u)) --pending[u];
        }
        CHECK(progress) << "the graph '" << name_ << "' has a cycle";
    }
    return out;
}

void Graph::MigrateNodes(const std::vector<Node*>& nodes, const std::vector<Value*>& temps, Graph* to) {
    auto take_node = [this](Node* n) {
        for (auto& up : all_nodes_)
            if (up.get() == n) return std::move(up);
        CHECK(false) << "node " << n->ToString() << " is not in graph '" << name_ << "'";
        return std::unique_ptr<Node>();
    };
    for (Node* n : nodes) {
        to->all_nodes_.push_back(take_node(n));
        to->nodes_.push_back(n);
        nodes_.erase(std::remove(nodes_.begin(), nodes_.end(), n), nodes_.end());
    }
    all_nodes_.erase(std::remove(all_nodes_.begin(), all_nodes_.end(), nullptr), all_nodes_.end());
    for (Value* v : temps) {
        for (auto& up : all_values_)
            if (up.get() == v) {
                to->all_values_.push_back(std::move(up));
                to->temp_values_.push_back(v);
            }
        temp_values_.erase(std::remove(temp_values_.begin(), temp_values_.end(), v), temp_values_.end());
    }
    all_values_.erase(std::remove(all_values_.begin(), all_values_.end(), nullptr), all_values_.end());
}

std::string Graph::GenSym(const std::string& base) {
    const int id = ++ids_[base];
    return base + "_" + std::to_string(id);
}

void Graph::CheckSanity(const std::string& where) const {
    std::set<const Value*> known;
    for (const auto& v : all_values_) known.insert(v.get());
    for (Node* n : GetLiveNodes()) {
        for (Value* v : n->inputs()) {
            CHECK(known.count(v)) << where << ": " << n->ToString() << " reads a value of another graph";
            CHECK(std::count(v->users().begin(), v->users().end(), n)) << where << ": user list of '" << v->name() << "' misses " << n->ToString();
        }
        for (Value* v : n->outputs()) {
            CHECK(known.count(v)) << where << ": " << n->ToString() << " writes a value of another graph";
            CHECK(v->IsNull() || v->producer() == n) << where << ": producer of '" << v->name() << "' is not " << n->ToString();
        }
    }
    for (Value* v : output_values_) CHECK(v->producer() || v->initializer()) << where << ": output '" << v->name() << "' has no producer";
    GetTopologicallySortedNodes();
}

std::string Graph::DebugString() const {
    std::ostringstream oss;
    for (Node* n : GetTopologicallySortedNodes()) {
        oss << n->ToString();
        if (n->subgraph()) {
            oss << " [" << n->fusion_type() << " #" << n->chainer_fusion_group() << ":";
            for (Node* s : n->subgraph()->GetTopologicallySortedNodes()) oss << " " << s->op_type();
            oss << "]";
        }
        oss << "\n";
    }
    return oss.str();
}

std::unique_ptr<Graph> Graph::FromOnnx(const OnnxGraph& x) {
    std::unique_ptr<Graph> g(new Graph(x.name));
    std::map<std::string, Value*> by_name;
    std::map<std::string, const OnnxValueInfo*> info;
    for (const OnnxValueInfo& vi : x.value_info) info[vi.name] = &vi;
    auto type_of = [](const OnnxValueInfo& vi) {
        Type t;
        t.dtype = DtypeFromOnnx(vi.elem_type);
        t.dims = vi.dims;
        t.has_dims = vi.has_shape;
        return t;
    };
    std::map<std::string, const OnnxTensor*> inits;
    for (const OnnxTensor& t : x.initializers) inits[t.name] = &t;
    for (const OnnxValueInfo& vi : x.inputs) {
        Value* v = g->AddInputValue(vi.name, type_of(vi));
        by_name[vi.name] = v;
        auto it = inits.find(vi.name);
        if (it != inits.end()) {
            v->ResetInitializer(std::make_unique<Tensor>(Tensor::FromOnnx(*it->second)));
            inits.erase(it);
        }
    }
    // initializers that are not listed as graph inputs (IR version 4 and later)
    for (const OnnxTensor& t : x.initializers) {
        if (!inits.count(t.name)) continue;
        Tensor tensor = Tensor::FromOnnx(t);
        Value* v = g->AddInputValue(t.name, Type(tensor.dtype(), tensor.dims()));
        v->ResetInitializer(std::make_unique<Tensor>(std::move(tensor)));
        by_name[t.name] = v;
    }
    for (const OnnxValueInfo& vi : x.outputs) by_name[vi.name] = g->AddOutputValue(vi.name, type_of(vi));
    auto get = [&](const std::string& name) -> Value* {
        if (name.empty()) return g->AddNullValue();
        auto it = by_name.find(name);
        if (it != by_name.end()) return it->second;
        Type t;
        auto vi = info.find(name);
        if (vi != info.end()) t = type_of(*vi->second);
        return by_name[name] = g->AddValue(name, t);
    };
    for (const OnnxNode& xn : x.nodes) {
        std::vector<Value*> ins, outs;
        for (const std::string& s : xn.inputs) ins.push_back(get(s));
        for (const std::string& s : xn.outputs) outs.push_back(get(s));
        Node* n = g->AddNode(xn.op_type, ins, outs, xn.name);
        n->attrs() = xn.attrs;
        n->set_domain(xn.domain);
    }
    return g;
}

OnnxGraph Graph::ToOnnx() const {
    OnnxGraph x;
    x.name = name_;
    auto info = [](const Value* v) {
        OnnxValueInfo vi;
        vi.name = v->name();
        vi.elem_type = DtypeToOnnx(v->type().dtype);
        vi.dims = v->type().dims;
        vi.has_shape = v->type().has_dims;
        return vi;
    };
    for (Value* v : input_values_) {
        x.inputs.push_back(info(v));
        if (v->initializer()) {
            OnnxTensor t = v->initializer()->ToOnnx();
            t.name = v->name();
            x.initializers.push_back(t);
        }
    }
    for (Value* v : output_values_) x.outputs.push_back(info(v));
    std::function<void(const Graph&, const std::map<const Value*, std::string>&)> emit;
    emit = [&](const Graph& g, const std::map<const Value*, std::string>& rename) {
        auto name_of = [&rename](const Value* v) {
            auto it = rename.find(v);
            return it != rename.end() ? it->second : v->name();
        };
        for (Node* n : g.GetTopologicallySortedNodes()) {
            if (n->subgraph()) {
                // a fusion group is written as the nodes it holds, on the outer values
                std::map<const Value*, std::string> inner;
                size_t k = 0;
                for (Value* v : n->subgraph()->input_values())
                    if (!v->initializer()) inner[v] = name_of(n->input(k++));
                for (size_t i = 0; i < n->outputs().size(); ++i) inner[n->subgraph()->output_values()[i]] = name_of(n->output(i));
                emit(*n->subgraph(), inner);
                continue;
            }
            OnnxNode xn;
            xn.op_type = n->op_type();
            xn.name = n->name();
            xn.domain = n->domain();
            for (Value* v : n->inputs()) xn.inputs.push_back(v->IsNull() ? "" : name_of(v));
            for (Value* v : n->outputs()) xn.outputs.push_back(v->IsNull() ? "" : name_of(v));
            xn.attrs = n->attrs();
            x.nodes.push_back(xn);
        }
    };
    emit(*this, {});
    return x;
}

// ---- GraphBuilder --------------------------------------------------------------------------------

GraphBuilder::GraphBuilder(Graph* graph, const std::string& category, Value* target)
    : graph_(graph), category_(category), target_name_(target ? target->name() : "") {
}

Value* GraphBuilder::Temp(const Type& type) {
    return graph_->AddValue(graph_->GenSym(category_ + "_" + target_name_), type);
}

Value* GraphBuilder::Op(const std::string& op_type, const std::vector<Value*>& inputs, Value* output) {
    if (!output) output = Temp();
    graph_->AddNode(op_type, inputs, {output}, category_);
    return output;
}

Node* GraphBuilder::MOp(const std::string& op_type, const std::vector<Value*>& inputs, const std::vector<Value*>& outputs) {
    return graph_->AddNode(op_type, inputs, outputs, category_);
}

Value* GraphBuilder::Const(const Tensor& tensor) {
    Value* v = Temp(Type(tensor.dtype(), tensor.dims()));
    Node* n = graph_->AddNode("Constant", {}, {v}, category_);
    n->SetTensor("value", tensor);
    return v;
}

// ---- InferDtypes ----------------------------------------------------------------------------------

void InferDtypes(Graph* graph) {
    auto dtype_of = [](const Value* v) {
        if (v->type().dtype != kUnknown) return v->type().dtype;
        if (v->initializer()) return v->initializer()->dtype();
        return kUnknown;
    };
    for (Node* n : graph->GetTopologicallySortedNodes()) {
        if (n->subgraph()) continue;
        const std::string& op = n->op_type();
        CDtype dt = kUnknown;
        auto zero_point_dtype = [&](size_t index) {
            if (index < n->inputs().size() && !n->input(static_cast<int>(index))->IsNull()) {
                const CDtype z = dtype_of(n->input(static_cast<int>(index)));
                if (z != kUnknown) return z;
            }
            return kUInt8;
        };
        if (op == "Constant") {
            std::unique_ptr<Tensor> t = n->tensor_value();
            if (t) dt = t->dtype();
        } else if (op == "QuantizeLinear") {
            dt = zero_point_dtype(2);
        } else if (op == "QLinearConv" || op == "QLinearMatMul") {
            dt = zero_point_dtype(7);
        } else if (op == "DequantizeLinear") {
            dt = kFloat32;
        } else if (op == "ConvInteger" || op == "MatMulInteger") {
            dt = kInt32;
        } else if (op == "Cast") {
            dt = DtypeFromOnnx(static_cast<int>(n->GetInt("to", 0)));
        } else if (!n->inputs().empty() && !n->input(0)->IsNull()) {
            dt = dtype_of(n->input(0));
        }
        // shapes, where they follow from the operands alone: a reduction over everything gives a 0-d
        // value, element-wise ops broadcast, the quantizing ops keep the shape of their first operand
        auto dims_of = [](const Value* v, std::vector<int64_t>* dims) {
            if (v->type().has_dims) {
                for (int64_t d : v->type().dims)
                    if (d < 0) return false;
                *dims = v->type().dims;
                return true;
            }
            if (v->initializer()) {
                *dims = v->initializer()->dims();
                return true;
            }
            return false;
        };
        static const std::set<std::string> unary = {"Identity", "Neg", "Abs", "Floor", "Round", "Exp", "Tanh", "Sigmoid", "Relu", "Cast", "Clip",
                                                    "QuantizeLinear", "DequantizeLinear"};
        static const std::set<std::string> binary = {"Add", "Sub", "Mul", "Div", "Max", "Min", "BitShift"};
        std::vector<int64_t> dims;
        bool has_dims = false;
        if (op == "Constant") {
            if (std::unique_ptr<Tensor> t = n->tensor_value()) {
                dims = t->dims();
                has_dims = true;
            }
        } else if ((op == "ReduceMin" || op == "ReduceMax") && n->GetInts("axes").empty() && n->GetInt("keepdims", 1) == 0) {
            has_dims = true;
        } else if (unary.count(op) && !n->inputs().empty() && !n->input(0)->IsNull()) {
            has_dims = dims_of(n->input(0), &dims);
        } else if (binary.count(op) && n->inputs().size() == 2) {
            std::vector<int64_t> a, b;
            if (dims_of(n->input(0), &a) && dims_of(n->input(1), &b)) {
                has_dims = true;
                const size_t rank = std::max(a.size(), b.size());
                dims.assign(rank, 1);
                for (size_t i = 0; i < rank && has_dims; ++i) {
                    const int64_t da = i < rank - a.size() ? 1 : a[i - (rank - a.size())];
                    const int64_t db = i < rank - b.size() ? 1 : b[i - (rank - b.size())];
                    if (da != db && da != 1 && db != 1) has_dims = false;
                    dims[i] = da == 1 ? db : da;
                }
            }
        }
        for (Value* o : n->outputs()) {
            if (o->IsNull()) continue;
            Type t = o->type();
            if (t.dtype == kUnknown) t.dtype = dt;
            if (!t.has_dims && has_dims) {
                t.dims = dims;
                t.has_dims = true;
            }
            o->set_type(t);
        }
    }
}

// ---- ClassifyValues ------------------------------------------------------------------------------

void ClassifyValues(const std::vector<Node*>& nodes, std::vector<Value*>* inputs, std::vector<Value*>* outputs, std::vector<Value*>* temps) {
    // values read from outside the set are inputs; values produced inside that somebody outside (or
    // the graph) still reads are outputs; the rest are temporaries
    std::set<Value*> temp_set, input_set;
    std::map<Value*, int> output_users;
    for (Node* node : nodes) {
        for (Value* v : node->inputs()) {
            input_set.insert(v);
            temp_set.insert(v);
        }
        for (Value* v : node->outputs()) {
            int users = static_cast<int>(v->users().size());
            if (v->IsOutput()) users = INT_MAX;
            CHECK(output_users.emplace(v, users).second) << v->name();
            temp_set.insert(v);
        }
    }
    for (Node* node : nodes)
        for (Value* v : node->inputs()) {
            auto found = output_users.find(v);
            if (found != output_users.end()) --found->second;
        }
    for (const auto& p : output_users) input_set.erase(p.first);
    inputs->assign(input_set.begin(), input_set.end());
    for (const auto& p : output_users) {
        CHECK_LE(0, p.second);
        if (p.second > 0) outputs->push_back(p.first);
    }
    for (Value* v : *inputs) temp_set.erase(v);
    for (Value* v : *outputs) temp_set.erase(v);
    temps->assign(temp_set.begin(), temp_set.end());
    auto by_name = [](const Value* a, const Value* b) { return a->name() < b->name(); };
    std::sort(inputs->begin(), inputs->end(), by_name);
    std::sort(outputs->begin(), outputs->end(), by_name);
    std::sort(temps->begin(), temps->end(), by_name);
}

}  // namespace chainer_compiler
