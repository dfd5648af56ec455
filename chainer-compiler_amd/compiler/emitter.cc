#include "emitter.h"

#include <algorithm>
#include <map>
#include <set>

#include "../runtime/log.h"
#include "fusion.h"

namespace chainer_compiler {

namespace {

using runtime::ChxVMInstructionProto;
using runtime::ChxVMProgramProto;
using runtime::ChxVMTypeProto;
using runtime::ChxVMValueProto;

ChxVMValueProto ArrayIn(int id) {
    ChxVMValueProto v;
    v.type = ChxVMValueProto::ARRAY;
    v.set_array(id);
    return v;
}
// an optional operand travels with the type of the plain one and the id -1 when absent
// (runtime/gen_chxvm.py:157-178 reads both through the same accessor)
ChxVMValueProto OptionalArrayIn(int id) {
    ChxVMValueProto v;
    v.type = ChxVMValueProto::ARRAY;
    v.set_array(id);
    return v;
}
ChxVMValueProto ArrayListIn(const std::vector<int>& ids) {
    ChxVMValueProto v;
    v.type = ChxVMValueProto::ARRAY_LIST;
    v.array_list.assign(ids.begin(), ids.end());
    return v;
}
ChxVMValueProto ScalarIn(int id, bool optional = false) {
    ChxVMValueProto v;
    (void)optional;
    v.type = ChxVMValueProto::SCALAR;
    v.set_scalar(id);
    return v;
}
ChxVMValueProto ShapeIn(int id) {
    ChxVMValueProto v;
    v.type = ChxVMValueProto::SHAPE;
    v.set_shape(id);
    return v;
}
ChxVMValueProto IntIn(int64_t i) {
    ChxVMValueProto v;
    v.type = ChxVMValueProto::INT;
    v.set_i(i);
    return v;
}
ChxVMValueProto FloatIn(double f) {
    ChxVMValueProto v;
    v.type = ChxVMValueProto::FLOAT;
    v.set_f(f);
    return v;
}
ChxVMValueProto IntsIn(const std::vector<int64_t>& ints, int type = ChxVMValueProto::INTS) {
    ChxVMValueProto v;
    v.type = type;
    v.ints = ints;
    return v;
}
ChxVMValueProto DoublesIn(const std::vector<double>& d) {
    ChxVMValueProto v;
    v.type = ChxVMValueProto::DOUBLES;
    v.doubles = d;
    return v;
}
ChxVMValueProto StringIn(const std::string& s) {
    ChxVMValueProto v;
    v.type = ChxVMValueProto::STRING;
    v.set_s(s);
    return v;
}

// positions of operands that the ops read through StrictScalar (runtime/chxvm_defs.py:451-471)
const std::map<std::string, std::set<int>>& ScalarOperands() {
    static const std::map<std::string, std::set<int>> m = {
            {"QuantizeLinear", {1, 2}}, {"DequantizeLinear", {1, 2}}, {"QLinearConv", {1, 2, 6, 7}},
            {"QLinearMatMul", {1, 2, 4, 5, 6, 7}}, {"ConvInteger", {2}}, {"Clip", {1, 2}}};
    return m;
}

class Emitter {
public:
    explicit Emitter(const Graph& graph) : graph_(graph) {
    }

    ChxVMProgramProto Run() {
        const std::vector<Node*> order = graph_.GetTopologicallySortedNodes();
        // which constants are read as scalars (and only as scalars)
        for (Node* n : order) {
            if (n->op_type() == "ChainerFusionGroup") {
                // only the operands of the kernel count; scale / zero-point / bound parameters are in the text
                GroupCode& gc = group_code_[n];
                gc.code = BuildHipProgram(*n, &gc.used);
                for (int i : gc.used) array_uses_.insert(n->input(i));
                continue;
            }
            auto it = ScalarOperands().find(n->op_type());
            for (size_t i = 0; i < n->inputs().size(); ++i) {
                Value* v = n->input(static_cast<int>(i));
                if (v->IsNull()) continue;
                const bool scalar = it != ScalarOperands().end() && it->second.count(static_cast<int>(i));
                (scalar ? scalar_uses_ : array_uses_).insert(v);
            }
        }
        for (Value* v : graph_.output_values()) array_uses_.insert(v);
        // last reader of every value, for Free
        for (size_t k = 0; k < order.size(); ++k)
            for (Value* v : order[k]->inputs())
                if (!v->IsNull()) last_use_[v] = static_cast<int>(k);

        for (Value* v : graph_.input_values()) {
            if (v->initializer()) {
                if (scalar_uses_.count(v) || array_uses_.count(v)) EmitConstant(v, *v->initializer());
                continue;
            }
            ChxVMInstructionProto* in = Add("In");
            in->inputs.push_back(StringIn(v->name()));
            in->outputs.push_back(IdOf(v));
            prog_.input_names.push_back(v->name());
            ChxVMTypeProto type;
            type.set_dtype(v->type().dtype);
            for (int64_t d : v->type().dims) type.shape.push_back(static_cast<int32_t>(d > 0 ? d : -1));
            prog_.input_types.push_back(type);
        }
        for (size_t k = 0; k < order.size(); ++k) {
            EmitNode(*order[k]);
            std::set<Value*> freed;
            for (Value* v : order[k]->inputs()) {
                if (v->IsNull() || v->IsOutput() || last_use_[v] != static_cast<int>(k) || !freed.insert(v).second) continue;
                if (!ids_.count(v)) continue;  // a parameter that was written into a statement, never materialised
                Add("Free")->inputs.push_back(ArrayIn(ids_[v]));
            }
        }
        for (Value* v : graph_.output_values()) {
            ChxVMInstructionProto* out = Add("Out");
            out->inputs.push_back(StringIn(v->name()));
            out->inputs.push_back(ArrayIn(IdOf(v)));
        }
        return std::move(prog_);
    }

private:
    int IdOf(Value* v) {
        auto it = ids_.find(v);
        if (it != ids_.end()) return it->second;
        return ids_[v] = next_id_++;
    }

    ChxVMInstructionProto* Add(const std::string& op, const std::string& debug_info = "") {
        const int number = runtime::OpNumber(op);
        CHECK(number > 0) << "no ChxVM op named " << op;
        prog_.instructions.emplace_back();
        ChxVMInstructionProto* inst = &prog_.instructions.back();
        inst->op = number;
        if (!debug_info.empty()) inst->set_debug_info(debug_info);
        inst->set_id(static_cast<int64_t>(prog_.instructions.size()));
        return inst;
    }

    // A constant tensor: a scalar constant when it has one element and every reader takes it as a
    // scalar, an array constant otherwise (the constant ops of runtime/ops/creation.cc:11-57).
    void EmitConstant(Value* v, const Tensor& t) {
        const bool is_float = DtypeIsFloat(t.dtype());
        if (t.NumElements() == 1 && scalar_uses_.count(v) && !array_uses_.count(v)) {
            ChxVMInstructionProto* c = Add(is_float ? "FloatScalarConstant" : "IntScalarConstant");
            c->inputs.push_back(is_float ? FloatIn(t.GetAsDouble(0)) : IntIn(static_cast<int64_t>(t.GetAsDouble(0))));
            c->inputs.push_back(IntIn(t.dtype()));
            c->inputs.push_back(IntIn(0));
            c->outputs.push_back(IdOf(v));
            return;
        }
        // read both ways: an array constant, which the scalar readers convert (runtime/chxvm_var.cc:70-76)
        ChxVMInstructionProto* c = Add(is_float ? "FloatConstant" : "IntConstant");
        if (is_float) {
            std::vector<double> values(t.NumElements());
            for (int64_t i = 0; i < t.NumElements(); ++i) values[i] = t.GetAsDouble(i);
            c->inputs.push_back(DoublesIn(values));
        } else {
            std::vector<int64_t> values(t.NumElements());
            for (int64_t i = 0; i < t.NumElements(); ++i) values[i] = static_cast<int64_t>(t.GetAsDouble(i));
            c->inputs.push_back(IntsIn(values, ChxVMValueProto::INT_VALUES));
        }
        c->inputs.push_back(IntIn(t.dtype()));
        c->inputs.push_back(IntsIn(t.dims()));
        c->inputs.push_back(IntIn(0));
        c->outputs.push_back(IdOf(v));
    }

    int Operand(const Node& n, size_t i, bool optional = false) {
        if (i >= n.inputs().size() || n.input(static_cast<int>(i))->IsNull()) {
            CHECK(optional) << n.ToString() << ": missing input " << i;
            return -1;
        }
        Value* v = n.input(static_cast<int>(i));
        CHECK(ids_.count(v)) << n.ToString() << ": input '" << v->name() << "' has not been computed";
        return ids_[v];
    }

    // strides, halved pads, group, auto_pad (compiler/chxvm/simple_node_emitter.cc:76-100)
    void ConvAttrs(const Node& n, ChxVMInstructionProto* inst) {
        for (int64_t d : n.GetInts("dilations")) CHECK_EQ(1, d) << "Dilation is not supported yet";
        const std::vector<int64_t> pads = n.GetInts("pads");
        CHECK_EQ(0UL, pads.size() % 2) << n.ToString();
        const size_t half = pads.size() / 2;
        for (size_t i = 0; i < half; ++i) CHECK_EQ(pads[i], pads[i + half]) << "paddings for beginning and end must be the same";
        std::string auto_pad = n.GetString("auto_pad", "NOTSET");
        if (auto_pad == "NOTSET") auto_pad = "";
        else CHECK(auto_pad == "SAME_UPPER") << "auto_pad " << auto_pad << " is not supported";
        inst->inputs.push_back(IntsIn(n.GetInts("strides")));
        inst->inputs.push_back(IntsIn(std::vector<int64_t>(pads.begin(), pads.begin() + half)));
        inst->inputs.push_back(IntIn(n.GetInt("group", 1)));
        inst->inputs.push_back(StringIn(auto_pad));
    }

    // The type a result is declared with, for the run-time check of every typed result
    // (compiler/chxvm/chxvm_value.cc:22-33): dtype and shape when both are known, else untyped.
    static ChxVMTypeProto TypeOf(const Value* v) {
        ChxVMTypeProto type;
        const Type& t = v->type();
        bool known = t.dtype != kUnknown && t.has_dims;
        for (int64_t d : t.dims) known = known && d > 0;  // 0 and -1 stand for an unknown extent
        if (known) {
            type.set_dtype(t.dtype);
            for (int64_t d : t.dims) type.shape.push_back(static_cast<int32_t>(d));
        }
        return type;
    }

    void EmitNode(const Node& n) {
        const std::string& op = n.op_type();
        const size_t nin = n.inputs().size();
        const std::string dbg = op + "(" + n.name() + ")";
        if (op == "Constant") {
            std::unique_ptr<Tensor> t = n.tensor_value();
            CHECK(t) << "Constant without a tensor value";
            // parameters that only fusion groups read were written into their program text
            if (!scalar_uses_.count(n.output(0)) && !array_uses_.count(n.output(0))) return;
            EmitConstant(n.output(0), *t);
            return;
        }
        if (op == "ChainerFusionGroup") {
            CHECK(n.fusion_type() == "hip" || n.fusion_type() == "nvrtc") << "fusion type " << n.fusion_type() << " has no emitter here";
            const GroupCode& gc = group_code_.at(&n);
            const std::string& code = gc.code;
            std::vector<int> ins;
            for (int i : gc.used) ins.push_back(Operand(n, i));
            ChxVMInstructionProto* inst = Add("ElementWiseNvrtc", dbg);
            inst->inputs.push_back(ArrayListIn(ins));
            inst->inputs.push_back(IntIn(static_cast<int64_t>(n.outputs().size())));
            inst->inputs.push_back(StringIn(code));
            inst->inputs.push_back(IntIn(n.chainer_fusion_group()));
            for (Value* o : n.outputs()) {
                inst->outputs.push_back(IdOf(o));
                inst->output_types.push_back(TypeOf(o));
                inst->output_names.push_back(o->name());
            }
            return;
        }
        CHECK_EQ(1UL, n.outputs().size()) << n.ToString();
        Value* out = n.output(0);
        auto simple = [&](const std::string& name, std::vector<ChxVMValueProto> inputs) {
            ChxVMInstructionProto* inst = Add(name, dbg);
            inst->inputs = std::move(inputs);
            inst->outputs.push_back(IdOf(out));
            inst->output_types.push_back(TypeOf(out));
            inst->output_names.push_back(out->name());  // names the per-op output dumps (compiler/chxvm/emitter.cc:72-77)
            return inst;
        };
        if ((op == "QuantizeLinear" || op == "DequantizeLinear") && nin >= 2 && nin <= 3) {
            simple(op, {ArrayIn(Operand(n, 0)), ScalarIn(Operand(n, 1)), ScalarIn(Operand(n, 2, true), true)});
        } else if (op == "QLinearConv" && nin >= 8 && nin <= 9) {
            ChxVMInstructionProto* inst = simple(op, {ArrayIn(Operand(n, 0)), ScalarIn(Operand(n, 1)), ScalarIn(Operand(n, 2)),
                                                      ArrayIn(Operand(n, 3)), ArrayIn(Operand(n, 4)), ArrayIn(Operand(n, 5)),
                                                      ScalarIn(Operand(n, 6)), ScalarIn(Operand(n, 7)), OptionalArrayIn(Operand(n, 8, true))});
            ConvAttrs(n, inst);
        } else if (op == "ConvInteger" && nin >= 2 && nin <= 4) {
            ChxVMInstructionProto* inst = simple(op, {ArrayIn(Operand(n, 0)), ArrayIn(Operand(n, 1)), ScalarIn(Operand(n, 2, true), true),
                                                      OptionalArrayIn(Operand(n, 3, true))});
            ConvAttrs(n, inst);
        } else if (op == "MatMulInteger" && nin >= 2 && nin <= 4) {
            simple(op, {ArrayIn(Operand(n, 0)), ArrayIn(Operand(n, 1)), OptionalArrayIn(Operand(n, 2, true)), OptionalArrayIn(Operand(n, 3, true))});
        } else if (op == "QLinearMatMul" && nin == 8) {
            // ReplaceQLinearMatMul, compiler/simplifier.cc:675-694
            const int a = next_id_++, b = next_id_++, mm = next_id_++;
            ChxVMInstructionProto* i1 = Add("DequantizeLinear", dbg);
            i1->inputs = {ArrayIn(Operand(n, 0)), ScalarIn(Operand(n, 1)), ScalarIn(Operand(n, 2), true)};
            i1->outputs.push_back(a);
            ChxVMInstructionProto* i2 = Add("DequantizeLinear", dbg);
            i2->inputs = {ArrayIn(Operand(n, 3)), ScalarIn(Operand(n, 4)), ScalarIn(Operand(n, 5), true)};
            i2->outputs.push_back(b);
            ChxVMInstructionProto* i3 = Add("MatMul", dbg);
            i3->inputs = {ArrayIn(a), ArrayIn(b)};
            i3->outputs.push_back(mm);
            simple("QuantizeLinear", {ArrayIn(mm), ScalarIn(Operand(n, 6)), ScalarIn(Operand(n, 7), true)});
            for (int tmp : {a, b, mm}) Add("Free")->inputs.push_back(ArrayIn(tmp));
        } else if ((op == "MaxPool" || op == "AveragePool") && nin == 1) {
            const std::vector<int64_t> pads = n.GetInts("pads");
            const size_t half = pads.size() / 2;
            for (size_t i = 0; i < half; ++i) CHECK_EQ(pads[i], pads[i + half]) << "paddings for beginning and end must be the same";
            const std::vector<int64_t> begin(pads.begin(), pads.begin() + half);
            ChxVMInstructionProto* inst;
            if (op == "MaxPool") {
                inst = simple(op, {ArrayIn(Operand(n, 0)), IntsIn(n.GetInts("kernel_shape")), IntsIn(n.GetInts("strides")), IntsIn(begin),
                                   IntIn(n.GetInt("chainer_cover_all", 0)), StringIn(n.GetString("auto_pad", "NOTSET"))});
            } else {
                inst = simple(op, {ArrayIn(Operand(n, 0)), IntsIn(n.GetInts("kernel_shape")), IntsIn(n.GetInts("strides")), IntsIn(begin),
                                   IntIn(n.GetInt("count_include_pad", 0))});
            }
            inst->outputs.push_back(-1);  // the backward context is not kept
            // an instruction that names its outputs names and types all of them (the run-time type check
            // compares the counts, runtime/chxvm.cc:38-64): the dropped context is nameless and untyped
            if (!inst->output_names.empty()) {
                inst->output_names.push_back("");
                inst->output_types.push_back(ChxVMTypeProto());
            }
        } else if ((op == "GlobalMaxPool" || op == "GlobalAveragePool") && nin == 1) {
            // ReplaceGlobalPool, compiler/simplifier.cc:272-290: the pool whose window is the input's spatial extent
            const Type& t = n.input(0)->type();
            bool known = t.has_dims;
            for (int64_t d : t.dims) known = known && d > 0;
            CHECK(known) << "The input shape of " << op << " must be known";
            CHECK_LT(2u, t.dims.size()) << "The input of " << op << " must have at least 3 dimensions";
            const std::vector<int64_t> kernel(t.dims.begin() + 2, t.dims.end());
            const std::vector<int64_t> ones(kernel.size(), 1), zeros(kernel.size(), 0);
            ChxVMInstructionProto* inst;
            if (op == "GlobalMaxPool") {
                inst = simple("MaxPool", {ArrayIn(Operand(n, 0)), IntsIn(kernel), IntsIn(ones), IntsIn(zeros), IntIn(0), StringIn("NOTSET")});
            } else {
                inst = simple("AveragePool", {ArrayIn(Operand(n, 0)), IntsIn(kernel), IntsIn(ones), IntsIn(zeros), IntIn(0)});
            }
            inst->outputs.push_back(-1);
            if (!inst->output_names.empty()) {
                inst->output_names.push_back("");
                inst->output_types.push_back(ChxVMTypeProto());
            }
        } else if (op == "Clip" && nin >= 1 && nin <= 3) {
            // compiler/chxvm/simple_node_emitter.cc:506-512: bounds as attributes or as operands
            if (nin == 1) {
                simple("StaticClip", {ArrayIn(Operand(n, 0)), FloatIn(n.GetFloat("max", 3.4028234663852886e38f)),
                                      FloatIn(n.GetFloat("min", -3.4028234663852886e38f))});
            } else {
                simple(op, {ArrayIn(Operand(n, 0)), ScalarIn(Operand(n, 1, true), true), ScalarIn(Operand(n, 2, true), true)});
            }
        } else if (op == "Max" || op == "Min") {
            std::vector<int> ins;
            for (size_t i = 0; i < nin; ++i) ins.push_back(Operand(n, i));
            simple(op, {ArrayListIn(ins)});
        } else if ((op == "ReduceMax" || op == "ReduceMin") && nin == 1) {
            simple(op, {ArrayIn(Operand(n, 0)), IntsIn(n.GetInts("axes")), IntIn(n.GetInt("keepdims", 1))});
        } else if (op == "MatMul" && nin == 2) {
            simple(op, {ArrayIn(Operand(n, 0)), ArrayIn(Operand(n, 1))});
        } else if (op == "Gemm" && (nin == 2 || nin == 3)) {
            // compiler/chxvm/simple_node_emitter.cc:316-318; attribute defaults of compiler/gen_node.py
            simple(op, {ArrayIn(Operand(n, 0)), ArrayIn(Operand(n, 1)), OptionalArrayIn(Operand(n, 2, true)), FloatIn(n.GetFloat("alpha", 1.f)),
                        FloatIn(n.GetFloat("beta", 1.f)), IntIn(n.GetInt("transA", 0)), IntIn(n.GetInt("transB", 0))});
        } else if (op == "Conv" && (nin == 2 || nin == 3)) {
            // compiler/chxvm/simple_node_emitter.cc:213-219: a convolution the quantizer did not rewrite
            ChxVMInstructionProto* inst = simple(op, {ArrayIn(Operand(n, 0)), ArrayIn(Operand(n, 1)), OptionalArrayIn(Operand(n, 2, true))});
            ConvAttrs(n, inst);
        } else if (op == "Concat" && nin >= 1) {
            std::vector<int> ins;  // compiler/chxvm/simple_node_emitter.cc:490-494
            for (size_t i = 0; i < nin; ++i) ins.push_back(Operand(n, i));
            simple(op, {ArrayListIn(ins), IntIn(n.GetInt("axis", 1))});
        } else if (op == "Transpose" && nin == 1) {
            simple(op, {ArrayIn(Operand(n, 0)), IntsIn(n.GetInts("perm"))});  // compiler/chxvm/simple_node_emitter.cc:523-526
        } else if (op == "Squeeze" && nin == 1) {
            simple(op, {ArrayIn(Operand(n, 0)), IntsIn(n.GetInts("axes"))});  // :297-300
        } else if (op == "Unsqueeze" && nin == 1) {
            // :301-311: the axes sorted; negative and positive ones together are refused
            std::vector<int64_t> axes = n.GetInts("axes");
            std::sort(axes.begin(), axes.end());
            if (!axes.empty()) CHECK(!(axes.front() < 0 && axes.back() > 0)) << "Unsqueeze with negative/positive axes mixed is not supported";
            simple(op, {ArrayIn(Operand(n, 0)), IntsIn(axes)});
        } else if (op == "Softmax" && nin == 1) {
            // compiler/chxvm/simple_node_emitter.cc:385-386; attribute defaults of compiler/gen_node.py:223
            simple(op, {ArrayIn(Operand(n, 0)), IntIn(n.GetInt("axis", 1)), IntIn(n.GetInt("chainer_is_onnx_semantics", 1))});
        } else if (op == "BatchNormalization" && nin == 5) {
            // EmitBatchNormalization, compiler/chxvm/emitter.cc:193-206: one output is the inference form
            CHECK_EQ(1, n.GetInt("spatial", 1)) << "`spatial` for BatchNormalization was removed from ONNX";
            CHECK_EQ(1u, n.outputs().size()) << "BatchNormalization with the outputs of a training step is not on the quantized-inference path";
            simple("FixedBatchNormalization", {ArrayIn(Operand(n, 0)), ArrayIn(Operand(n, 1)), ArrayIn(Operand(n, 2)), ArrayIn(Operand(n, 3)),
                                               ArrayIn(Operand(n, 4)), FloatIn(n.GetFloat("epsilon", 1e-5f))});
        } else if (op == "Flatten" && nin == 1) {
            // compiler/chxvm/simple_node_emitter.cc:698-701
            simple(op, {ArrayIn(Operand(n, 0)), IntIn(n.GetInt("axis", 1))});
        } else if (op == "Reshape" && nin == 2) {
            simple(op, {ArrayIn(Operand(n, 0)), ShapeIn(Operand(n, 1))});
        } else if (op == "Cast" && nin == 1) {
            const CDtype to = DtypeFromOnnx(static_cast<int>(n.GetInt("to", 0)));
            CHECK(to != kUnknown) << n.ToString() << ": unsupported target type " << n.GetInt("to", 0);
            simple(op, {ArrayIn(Operand(n, 0)), IntIn(to)});
        } else if (op == "Identity" || op == "Neg" || op == "Exp" || op == "Tanh" || op == "Sigmoid" || op == "Relu" || op == "Abs" ||
                   op == "Floor" || op == "Round") {
            CHECK_EQ(1UL, nin) << n.ToString();
            simple(op, {ArrayIn(Operand(n, 0))});
        } else if (op == "Add" || op == "Sub" || op == "Mul" || op == "Div") {
            CHECK_EQ(2UL, nin) << n.ToString();
            simple(op, {ArrayIn(Operand(n, 0)), ArrayIn(Operand(n, 1))});
        } else if (op == "BitShift") {
            // compiler/chxvm/simple_node_emitter.cc:681-684
            CHECK_EQ(2UL, nin) << n.ToString();
            simple(op, {ArrayIn(Operand(n, 0)), ArrayIn(Operand(n, 1)), StringIn(n.GetString("direction", ""))});
        } else {
            CHECK(false) << "node type " << op << " (" << nin << " inputs) is not on the quantized-inference path";
        }
    }

    struct GroupCode {
        std::string code;
        std::vector<int> used;
    };
    std::map<const Node*, GroupCode> group_code_;
    const Graph& graph_;
    ChxVMProgramProto prog_;
    std::map<Value*, int> ids_;
    std::map<Value*, int> last_use_;
    std::set<Value*> scalar_uses_, array_uses_;
    int next_id_ = 1;
};

}  // namespace

runtime::ChxVMProgramProto EmitProgram(const Graph& graph) {
    return Emitter(graph).Run();
}

}  // namespace chainer_compiler
