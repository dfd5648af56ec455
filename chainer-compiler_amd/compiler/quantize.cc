#include "quantize.h"

#include <algorithm>
#include <cmath>

#include "../runtime/log.h"

namespace chainer_compiler {

namespace {

struct Context : public QuantizationOptions {
    explicit Context(const QuantizationOptions& o) : QuantizationOptions(o) {
    }
    Graph* graph = nullptr;
    CDtype input_qdtype = kUInt8, weight_qdtype = kUInt8;
};

// one operand after quantization: the 8-bit value and the values holding its scale and zero point
struct QuantizedInput {
    Value* input;
    Value* scale;
    Value* zero_point;
    std::vector<int64_t> scale_zero_shape;  // per-channel: [OC, 1, 1, ...] for the scale-back multiply
};

float QRange(CDtype dt) {
    return dt == kUInt8 ? 255.f : 254.f;
}

Tensor ScalarTensor(float v) {
    return Tensor::FromVector<float>("", kFloat32, {}, {v});
}

Tensor DtypeScalarTensor(CDtype dt, int64_t v) {
    if (dt == kInt8) return Tensor::FromVector<int8_t>("", dt, {}, {static_cast<int8_t>(v)});
    CHECK_EQ(kUInt8, dt);
    return Tensor::FromVector<uint8_t>("", dt, {}, {static_cast<uint8_t>(v)});
}

Tensor CodesTensor(CDtype dt, const std::vector<int64_t>& dims, const std::vector<int32_t>& codes) {
    std::string raw(codes.size(), '\0');
    for (size_t i = 0; i < codes.size(); ++i) raw[i] = static_cast<char>(codes[i]);  // two's complement / modulo 256, as AsType
    return Tensor("", dt, dims, raw);
}

std::unique_ptr<Tensor> ConstTensorOf(const Value* v) {
    if (v->initializer()) return std::make_unique<Tensor>(*v->initializer());
    if (v->producer() && v->producer()->op_type() == "Constant") return v->producer()->tensor_value();
    return nullptr;
}

QuantizedInput QuantizeWeight(GraphBuilder* gb, const Tensor& w, CDtype dtype) {
    const QuantizedData q = QuantizeData(w.AsFloats(), dtype);
    return {gb->Const(CodesTensor(dtype, w.dims(), q.data)), gb->Const(ScalarTensor(q.scale)), gb->Const(DtypeScalarTensor(dtype, q.zero_point)), {}};
}

QuantizedInput QuantizeWeightConvolution(const Context& ctx, GraphBuilder* gb, const Tensor& w, CDtype dtype) {
    if (!ctx.per_channel) return QuantizeWeight(gb, w, dtype);
    // every output channel on its own range; the parameters become [OC] vectors
    const int64_t channels = w.dims().at(0), per = w.NumElements() / channels;
    const std::vector<float> all = w.AsFloats();
    std::vector<float> scales;
    std::vector<int32_t> zero_points, codes;
    for (int64_t c = 0; c < channels; ++c) {
        const QuantizedData q = QuantizeData(std::vector<float>(all.begin() + c * per, all.begin() + (c + 1) * per), dtype);
        scales.push_back(q.scale);
        zero_points.push_back(static_cast<int32_t>(q.zero_point));
        codes.insert(codes.end(), q.data.begin(), q.data.end());
    }
    std::vector<int64_t> param_shape = {channels};
    Value* scale = gb->Const(Tensor::FromVector<float>("", kFloat32, param_shape, scales));
    Value* zero_point = gb->Const(CodesTensor(dtype, param_shape, zero_points));
    for (size_t i = 2; i < w.dims().size(); ++i) param_shape.push_back(1);
    return {gb->Const(CodesTensor(dtype, w.dims(), codes)), scale, zero_point, param_shape};
}

std::vector<QuantizedInput> QuantizeInputs(const Context& ctx, GraphBuilder* gb, Node* node, const std::vector<int>& indices, int weight_index) {
    CHECK(node->op_type() == "Conv" || node->op_type() == "MatMul");
    std::vector<QuantizedInput> result;
    for (int index : indices) {
        const CDtype qtype = index == weight_index ? ctx.weight_qdtype : ctx.input_qdtype;
        Value* operand = node->input(index);
        if (std::unique_ptr<Tensor> constant = ConstTensorOf(operand)) {
            // an operand with a constant behind it is a weight
            if (node->op_type() == "Conv" && index == weight_index) result.push_back(QuantizeWeightConvolution(ctx, gb, *constant, qtype));
            else result.push_back(QuantizeWeight(gb, *constant, qtype));
            continue;
        }
        Value* scale;
        Value* zero_point;
        if (ctx.is_static) {
            auto it = ctx.input_quantization_params.find(operand->name());
            CHECK(it != ctx.input_quantization_params.end()) << "no quantization parameters for input '" << operand->name() << "'";
            scale = gb->Const(ScalarTensor(it->second.scale));
            zero_point = gb->Const(DtypeScalarTensor(qtype, it->second.zero_point));
        } else {
            // the parameters are computed from the tensor at run time
            Value* rmin = gb->Op("ReduceMin", {operand});
            rmin->producer()->SetInt("keepdims", 0);
            Value* rmax = gb->Op("ReduceMax", {operand});
            rmax->producer()->SetInt("keepdims", 0);
            Value* qrange = gb->Const(ScalarTensor(QRange(qtype)));
            if (qtype == kInt8) {
                Value* abs_max = gb->Op("Max", {gb->Op("Abs", {rmin}), gb->Op("Abs", {rmax})});
                scale = gb->Op("Div", {abs_max, qrange});
                zero_point = gb->Const(DtypeScalarTensor(qtype, 0));
            } else {
                scale = gb->Op("Div", {gb->Op("Sub", {rmax, rmin}), qrange});
                Value* zp_float = gb->Op("Floor", {gb->Op("Div", {gb->Op("Sub", {gb->Const(ScalarTensor(0.f)), rmin}), scale})});
                zero_point = gb->Op("Cast", {zp_float});
                zero_point->producer()->SetInt("to", DtypeToOnnx(qtype));
                zero_point->set_type(Type(qtype, {}));
            }
            scale->set_type(Type(kFloat32, {}));
        }
        Value* q = gb->Op("QuantizeLinear", {operand, scale, zero_point});
        q->set_type(Type(qtype, operand->type().dims));
        if (!operand->type().has_dims) q->set_type([&] { Type t; t.dtype = qtype; return t; }());
        result.push_back({q, scale, zero_point, {}});
    }
    return result;
}

const std::vector<std::string> kConvAttrs = {"dilations", "group", "kernel_shape", "strides", "auto_pad", "pads"};

Type Untyped(CDtype dt) {
    Type t;
    t.dtype = dt;
    return t;
}

// x_scale * w_scale (reshaped to [OC,1,1] when per channel) times the float copy of the int32 result
void ScaleBack(GraphBuilder* gb, const std::vector<QuantizedInput>& q, Value* int_out, Value* output) {
    Value* cast = gb->Op("Cast", {int_out});
    cast->producer()->SetInt("to", kOnnxFloat);
    cast->set_type(Untyped(kFloat32));
    Value* scales = gb->Op("Mul", {q[0].scale, q[1].scale});
    scales->set_type(Untyped(kFloat32));
    if (!q[1].scale_zero_shape.empty()) {
        Value* shape = gb->Const(Tensor::FromVector<int64_t>("", kInt64, {static_cast<int64_t>(q[1].scale_zero_shape.size())}, q[1].scale_zero_shape));
        scales = gb->Op("Reshape", {scales, shape});
        scales->set_type(Type(kFloat32, q[1].scale_zero_shape));
    }
    gb->Op("Mul", {cast, scales}, output);
}

void QuantizeWithIntegerOp(const Context& ctx, Node* node) {
    const bool conv = node->op_type() == "Conv";
    GraphBuilder gb(ctx.graph, conv ? "QuantizeConvWithInteger" : "QuantizeMatMulWithInteger", node->input(0));
    const std::vector<QuantizedInput> q = QuantizeInputs(ctx, &gb, node, {0, 1}, 1);
    Value* int_out = gb.Op(conv ? "ConvInteger" : "MatMulInteger", {q[0].input, q[1].input, q[0].zero_point, q[1].zero_point});
    int_out->set_type(Untyped(kInt32));
    if (conv) int_out->producer()->CopyAttrsFrom(*node, kConvAttrs);
    Value* output = node->output(0);
    ctx.graph->DetachNode(node);
    ScaleBack(&gb, q, int_out, output);
}

void QuantizeWithQLinearOp(const Context& ctx, Node* node) {
    const bool conv = node->op_type() == "Conv";
    GraphBuilder gb(ctx.graph, conv ? "QuantizeConvWithQLinear" : "QuantizeMatMulWithQLinear", node->input(0));
    const std::vector<QuantizedInput> q = QuantizeInputs(ctx, &gb, node, {0, 1}, 1);
    Value* output = node->output(0);
    auto it = ctx.output_quantization_params.find(output->name());
    CHECK(it != ctx.output_quantization_params.end()) << "no quantization parameters for output '" << output->name() << "'";
    Value* y_scale = gb.Const(ScalarTensor(it->second.scale));
    Value* y_zero_point = gb.Const(DtypeScalarTensor(it->second.zero_point_dtype, it->second.zero_point));
    Value* q_out = gb.Op(conv ? "QLinearConv" : "QLinearMatMul",
                         {q[0].input, q[0].scale, q[0].zero_point, q[1].input, q[1].scale, q[1].zero_point, y_scale, y_zero_point});
    q_out->set_type(Untyped(it->second.zero_point_dtype));
    if (conv) q_out->producer()->CopyAttrsFrom(*node, kConvAttrs);
    ctx.graph->DetachNode(node);
    gb.Op("DequantizeLinear", {q_out, y_scale, y_zero_point}, output);
}

}  // namespace

QuantizedData QuantizeData(const std::vector<float>& data, CDtype qtype) {
    QuantizedData q;
    float lo = 0.f, hi = 0.f;  // the range always contains 0
    for (float v : data) {
        lo = std::min(lo, v);
        hi = std::max(hi, v);
    }
    q.rmin = lo;
    q.rmax = hi;
    const float range = QRange(qtype);
    q.data.resize(data.size());
    // codes: rint in double of the float quotient (runtime/chainerx_util.cc:397-410), then the
    // float sum with the zero point, then a truncating cast
    if (qtype == kInt8) {
        const float max_range = std::max(std::fabs(lo), std::fabs(hi));
        q.scale = max_range * 2 / range;
        q.zero_point = 0;
        for (size_t i = 0; i < data.size(); ++i) {
            const float quotient = data[i] / q.scale;
            q.data[i] = q.scale == 0.f ? 0 : static_cast<int32_t>(static_cast<float>(std::rint(static_cast<double>(quotient))));
        }
    } else {
        CHECK_EQ(kUInt8, qtype);
        q.scale = lo != hi ? (hi - lo) / range : 1.f;
        q.zero_point = static_cast<int64_t>(std::rint((0 - lo) / q.scale));
        for (size_t i = 0; i < data.size(); ++i) {
            const float quotient = data[i] / q.scale;
            const float shifted = static_cast<float>(std::rint(static_cast<double>(quotient))) + static_cast<float>(q.zero_point);
            q.data[i] = static_cast<int32_t>(shifted);
        }
    }
    return q;
}

bool Quantize(const QuantizationOptions& opts, Graph* graph) {
    CHECK_EQ(8, opts.nbits);
    Context ctx(opts);
    ctx.graph = graph;
    ctx.input_qdtype = kUInt8;
    ctx.weight_qdtype = opts.asymmertic_input_types ? kInt8 : kUInt8;
    bool result = false;
    for (Node* node : graph->GetLiveNodes()) {
        if (node->op_type() == "Conv") {
            if (node->inputs().size() > 2) continue;  // a bias is not supported, the node stays float
        } else if (node->op_type() != "MatMul") {
            continue;
        }
        if (ctx.mode == QuantizationMode::IntegerOps) QuantizeWithIntegerOp(ctx, node);
        else QuantizeWithQLinearOp(ctx, node);
        result = true;
    }
    return result;
}

int ExpandDynamicQuantizeLinear(Graph* graph) {
    int replaced = 0;
    for (Node* node : graph->GetLiveNodes()) {
        if (node->op_type() != "DynamicQuantizeLinear") continue;
        CHECK_EQ(1UL, node->inputs().size()) << node->ToString();
        CHECK_EQ(3UL, node->outputs().size()) << node->ToString();
        Value* x = node->input(0);
        Value* const y = node->output(0);
        Value* const y_scale = node->output(1);
        Value* const y_zero_point = node->output(2);
        GraphBuilder gb(graph, "ExpandDynamicQuantizeLinear", y);
        graph->DetachNode(node);  // its outputs get new producers below
        auto reduce = [&](const char* op) {
            Value* v = gb.Op(op, {x});
            v->producer()->SetInt("keepdims", 0);
            return v;
        };
        Value* q_min = gb.Const(ScalarTensor(0.f));
        Value* q_max = gb.Const(ScalarTensor(255.f));
        Value* x_min_adjusted = gb.Op("Min", {reduce("ReduceMin"), q_min});
        Value* x_max_adjusted = gb.Op("Max", {reduce("ReduceMax"), q_min});
        Value* scale = gb.Op("Div", {gb.Op("Sub", {x_max_adjusted, x_min_adjusted}), q_max});
        Value* initial_zero_point = gb.Op("Sub", {q_min, gb.Op("Div", {x_min_adjusted, scale})});
        Value* rounded = gb.Op("Round", {gb.Op("Clip", {initial_zero_point, q_min, q_max})});
        Value* zero_point = gb.Op("Cast", {rounded});
        zero_point->producer()->SetInt("to", DtypeToOnnx(kUInt8));
        zero_point->set_type(Type(kUInt8, {}));
        scale->set_type(Type(kFloat32, {}));
        gb.Op("Identity", {scale}, y_scale);
        gb.Op("Identity", {zero_point}, y_zero_point);
        gb.Op("QuantizeLinear", {x, scale, zero_point}, y);
        ++replaced;
    }
    return replaced;
}

}  // namespace chainer_compiler
