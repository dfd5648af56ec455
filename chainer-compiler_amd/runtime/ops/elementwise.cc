// ElementWiseNvrtcOp::RunImpl on the hip backend (runtime/ops/nvrtc.cc:90-161 of the
// chainer-compiler tree): result shape = broadcast of the inputs, outputs allocated here, the
// kernel generated, compiled, cached and launched behind chx_hip_elementwise.  The inputs are
// handed over as they are; nothing is broadcast or copied first.
#include <cstdio>
#include <cstring>
#include <sstream>

#include "../gen/gen_chxvm_ops.h"

namespace chainer_compiler {
namespace runtime {

chainerx::Array AsContiguous(const chainerx::Array& a);  // ops/connection.cc

namespace {

// dtypes of the outputs: those the program declares (either form of program text: this library's, or the CUDA C
// that the reference's compiler emits, whose results have the type of its `typedef ... T`)
std::vector<chainerx::Dtype> OutputDtypes(const std::string& code) {
    int32_t codes[64];
    int32_t count = 0;
    CHXVM_HIP_CALL(chx_hip_elementwise_output_dtypes(code.c_str(), codes, 64, &count));
    CHECK_LE(count, 64) << "a fusion program with more than 64 outputs";
    std::vector<chainerx::Dtype> out;
    for (int32_t i = 0; i < count; ++i) out.push_back(static_cast<chainerx::Dtype>(codes[i]));
    return out;
}

}  // namespace

std::vector<chainerx::Array> ElementWiseNvrtcOp::RunImpl(ChxVMState* st, const std::vector<chainerx::Array>& orig_inputs) {
    CHECK(!orig_inputs.empty());
    chainerx::Shape shape = orig_inputs[0].shape();
    for (const chainerx::Array& input : orig_inputs) shape = chainerx::internal::BroadcastShapes(shape, input.shape());
    const std::vector<chainerx::Dtype> dtypes = OutputDtypes(code);
    CHECK_EQ(static_cast<size_t>(num_outputs), dtypes.size()) << "fusion program declares a different number of outputs";

    // channels-last operands give channels-last results, so chains between convolutions never transpose
    bool channels_last = shape.size() == 4;
    for (const chainerx::Array& input : orig_inputs)
        if (input.shape() == shape && (input.IsContiguous() || input.strides()[1] != input.GetItemSize())) channels_last = false;

    // Activations whose pixel pitch is padded to 16 bytes (a convolution's output with C = 24, say):
    // when every operand has that one layout and all values are 8-bit, the group runs over the padded
    // pixels as they lie in memory, which is dense; the padding bytes compute garbage into padding.
    bool padded = channels_last;
    for (const chainerx::Array& input : orig_inputs)
        padded = padded && input.shape() == shape && input.GetItemSize() == 1 && input.strides() == orig_inputs[0].strides() &&
                 input.strides()[3] > shape[1] && input.strides()[2] == shape[3] * input.strides()[3] &&
                 input.strides()[0] == shape[2] * input.strides()[2];
    for (chainerx::Dtype dt : dtypes) padded = padded && chainerx::GetItemSize(dt) == 1;
    const int64_t pitch = padded ? orig_inputs[0].strides()[3] : 0;
    padded = padded && pitch == (shape[1] + 15) / 16 * 16;
    auto widened = [&](chx_hip_tensor t) {
        if (padded) t.shape[1] = pitch;
        return t;
    };

    std::vector<chainerx::Array> outputs;
    std::vector<chx_hip_tensor> in_desc, out_desc;
    for (const chainerx::Array& input : orig_inputs) in_desc.push_back(widened(input.hip()));
    for (int i = 0; i < num_outputs; ++i) {
        outputs.push_back(padded          ? chainerx::EmptyChannelsLastPadded(shape, dtypes[i])
                          : channels_last ? chainerx::EmptyChannelsLast(shape, dtypes[i])
                                          : chainerx::Empty(shape, dtypes[i]));
        out_desc.push_back(widened(outputs.back().hip()));
    }
    std::vector<const chx_hip_tensor*> in_ptr;
    std::vector<chx_hip_tensor*> out_ptr;
    for (chx_hip_tensor& t : in_desc) in_ptr.push_back(&t);
    for (chx_hip_tensor& t : out_desc) out_ptr.push_back(&t);
    CHXVM_HIP_CALL(chx_hip_elementwise(code.c_str(), fusion_id, in_ptr.data(), static_cast<int32_t>(in_ptr.size()), out_ptr.data(),
                                       static_cast<int32_t>(out_ptr.size()), chainerx::CurrentStream()));
    return outputs;
}

// The float element-wise ops that stay single instructions when no fusion group takes them
// (runtime/ops/math.cc:31-41,105, activation.cc:20-22,55-61 of the chainer-compiler tree): each runs
// as a one-statement program through the same generator, so a value computed by a lone op and the
// same value computed inside a group are the same bits.
namespace {

chainerx::Array RunFloatOp(const char* op, const std::vector<chainerx::Array>& inputs) {
    static const char* names[] = {"a", "b"};
    chainerx::Shape shape = inputs[0].shape();
    std::string code = "chxhip-fusion 1\nin";
    for (size_t i = 0; i < inputs.size(); ++i) {
        CHECK(inputs[i].dtype() == chainerx::Dtype::kFloat32) << op << " runs on float32 arrays on the hip backend, got " << inputs[i].dtype();
        shape = chainerx::internal::BroadcastShapes(shape, inputs[i].shape());
        code += std::string(" ") + names[i] + ":float32";
    }
    code += std::string("\ny = ") + op;
    for (size_t i = 0; i < inputs.size(); ++i) code += std::string(" ") + names[i];
    code += "\nout y:float32\n";
    chainerx::Array y = chainerx::Empty(shape, chainerx::Dtype::kFloat32);
    std::vector<chx_hip_tensor> in_desc;
    for (const chainerx::Array& a : inputs) in_desc.push_back(a.hip());
    chx_hip_tensor out_desc = y.hip();
    std::vector<const chx_hip_tensor*> in_ptr;
    for (chx_hip_tensor& t : in_desc) in_ptr.push_back(&t);
    chx_hip_tensor* out_ptr = &out_desc;
    CHXVM_HIP_CALL(chx_hip_elementwise(code.c_str(), 0, in_ptr.data(), static_cast<int32_t>(in_ptr.size()), &out_ptr, 1, chainerx::CurrentStream()));
    return y;
}

}  // namespace

chainerx::Array AddOp::RunImpl(ChxVMState* st, const chainerx::Array& a, const chainerx::Array& b) {
    return RunFloatOp("Add", {a, b});
}
chainerx::Array SubOp::RunImpl(ChxVMState* st, const chainerx::Array& a, const chainerx::Array& b) {
    return RunFloatOp("Sub", {a, b});
}
chainerx::Array MulOp::RunImpl(ChxVMState* st, const chainerx::Array& a, const chainerx::Array& b) {
    return RunFloatOp("Mul", {a, b});
}
chainerx::Array DivOp::RunImpl(ChxVMState* st, const chainerx::Array& a, const chainerx::Array& b) {
    return RunFloatOp("Div", {a, b});
}
chainerx::Array NegOp::RunImpl(ChxVMState* st, const chainerx::Array& x) {
    return RunFloatOp("Neg", {x});
}
chainerx::Array ExpOp::RunImpl(ChxVMState* st, const chainerx::Array& x) {
    return RunFloatOp("Exp", {x});
}
chainerx::Array TanhOp::RunImpl(ChxVMState* st, const chainerx::Array& x) {
    return RunFloatOp("Tanh", {x});
}
chainerx::Array SigmoidOp::RunImpl(ChxVMState* st, const chainerx::Array& x) {
    return RunFloatOp("Sigmoid", {x});
}
chainerx::Array ReluOp::RunImpl(ChxVMState* st, const chainerx::Array& x) {
    return RunFloatOp("Relu", {x});
}
chainerx::Array AbsOp::RunImpl(ChxVMState* st, const chainerx::Array& x) {
    return RunFloatOp("Abs", {x});
}
chainerx::Array FloorOp::RunImpl(ChxVMState* st, const chainerx::Array& x) {
    return RunFloatOp("Floor", {x});
}
// ties to even (runtime/ops/quantize.cc:148-151, SlowRound)
chainerx::Array RoundOp::RunImpl(ChxVMState* st, const chainerx::Array& x) {
    return RunFloatOp("Round", {x});
}

namespace {

// Minimum(Maximum(x, lo), hi) with the bounds written into the program (runtime/ops/math.cc:140-154);
// a missing bound is the end of the float range, which changes no finite value
chainerx::Array ClipTo(const chainerx::Array& x, float lo, float hi) {
    CHECK(x.dtype() == chainerx::Dtype::kFloat32) << "Clip runs on float32 arrays on the hip backend, got " << x.dtype();
    uint32_t lo_bits, hi_bits;
    std::memcpy(&lo_bits, &lo, 4);
    std::memcpy(&hi_bits, &hi, 4);
    char line[96];
    std::snprintf(line, sizeof(line), "y = Clip a 0x%08x 0x%08x\n", lo_bits, hi_bits);
    const std::string code = std::string("chxhip-fusion 1\nin a:float32\n") + line + "out y:float32\n";
    chainerx::Array y = chainerx::Empty(x.shape(), chainerx::Dtype::kFloat32);
    chx_hip_tensor in_desc = x.hip(), out_desc = y.hip();
    const chx_hip_tensor* in_ptr = &in_desc;
    chx_hip_tensor* out_ptr = &out_desc;
    CHXVM_HIP_CALL(chx_hip_elementwise(code.c_str(), 0, &in_ptr, 1, &out_ptr, 1, chainerx::CurrentStream()));
    return y;
}

constexpr float kFloatMax = 3.4028234663852886e38f;

}  // namespace

chainerx::Array StaticClipOp::RunImpl(ChxVMState* st, const chainerx::Array& x) {
    return ClipTo(x, min, max);
}
// the operands arrive as (x, min, max): the emitter passes the node's inputs in their order
// (compiler/chxvm/simple_node_emitter.cc:511, runtime/ops/math.cc:144-154)
chainerx::Array ClipOp::RunImpl(
        ChxVMState* st, const chainerx::Array& x, const absl::optional<StrictScalar>& min, const absl::optional<StrictScalar>& max) {
    return ClipTo(x, min.has_value() ? static_cast<float>(*min) : -kFloatMax, max.has_value() ? static_cast<float>(*max) : kFloatMax);
}

// Maximum / Minimum folded over the operands (runtime/ops/math.cc:179-195)
chainerx::Array MaxOp::RunImpl(ChxVMState* st, const std::vector<chainerx::Array>& inputs) {
    CHECK_LT(0UL, inputs.size());
    chainerx::Array result = inputs[0];
    for (size_t i = 1; i < inputs.size(); ++i) result = RunFloatOp("Max", {result, inputs[i]});
    return result;
}
chainerx::Array MinOp::RunImpl(ChxVMState* st, const std::vector<chainerx::Array>& inputs) {
    CHECK_LT(0UL, inputs.size());
    chainerx::Array result = inputs[0];
    for (size_t i = 1; i < inputs.size(); ++i) result = RunFloatOp("Min", {result, inputs[i]});
    return result;
}

namespace {

// every axis reduced and dropped: the form the quantizer emits (compiler/quantize.cc:171-174)
chainerx::Array ReduceAll(const chainerx::Array& x, const chainerx::StackVector<int64_t, chainerx::kMaxNdim>& axes, int keepdims, bool is_max) {
    CHECK(axes.empty() || static_cast<int>(axes.size()) == x.ndim()) << "only the reduction over all axes runs on the hip backend";
    CHECK_EQ(0, keepdims) << "keepdims is not supported on the hip backend";
    CHECK(x.dtype() == chainerx::Dtype::kFloat32) << "ReduceMin / ReduceMax run on float32 arrays on the hip backend";
    chainerx::Array y = chainerx::Empty(chainerx::Shape{}, chainerx::Dtype::kFloat32);
    chx_hip_tensor xt = x.hip(), yt = y.hip();
    CHXVM_HIP_CALL(chx_hip_reduce_min_max(&xt, is_max ? 1 : 0, &yt, chainerx::CurrentStream()));
    return y;
}

}  // namespace

chainerx::Array ReduceMaxOp::RunImpl(ChxVMState* st, const chainerx::Array& x) {
    return ReduceAll(x, axes, keepdims, true);
}
chainerx::Array ReduceMinOp::RunImpl(ChxVMState* st, const chainerx::Array& x) {
    return ReduceAll(x, axes, keepdims, false);
}

// x.AsType(to) (runtime/ops/manipulation.cc:157-159)
chainerx::Array CastOp::RunImpl(ChxVMState* st, const chainerx::Array& input) {
    const chainerx::Dtype dt = static_cast<chainerx::Dtype>(to);
    if (dt == input.dtype()) return input;
    chainerx::Array y = chainerx::Empty(input.shape(), dt);
    chx_hip_tensor xt = input.hip(), yt = y.hip();
    CHXVM_HIP_CALL(chx_hip_cast(&xt, &yt, chainerx::CurrentStream()));
    return y;
}

// chainerx::LeftShift / RightShift over the broadcast of x and y (runtime/ops/quantize.cc:153-163)
chainerx::Array BitShiftOp::RunImpl(ChxVMState* st, const chainerx::Array& x, const chainerx::Array& y) {
    CHECK(chainerx::GetKind(x.dtype()) != chainerx::DtypeKind::kFloat) << "BitShift of " << x.dtype();
    CHECK(chainerx::GetKind(y.dtype()) != chainerx::DtypeKind::kFloat) << "BitShift by " << y.dtype();
    CHECK(direction == "LEFT" || direction == "RIGHT") << "BitShift direction " << direction;
    chainerx::Array z = chainerx::Empty(chainerx::internal::BroadcastShapes(x.shape(), y.shape()), x.dtype());
    chx_hip_tensor xt = x.hip(), yt = y.hip(), zt = z.hip();
    CHXVM_HIP_CALL(chx_hip_bit_shift(&xt, &yt, direction == "LEFT" ? 1 : 0, &zt, chainerx::CurrentStream()));
    return z;
}

// a view of the same memory, after a dense copy where the array is not dense (runtime/ops/manipulation.cc:30-53);
// -1 and 0 entries as ONNX defines them
chainerx::Array ReshapeOp::RunImpl(ChxVMState* st, const chainerx::Array& data, const chainerx::Shape& shape) {
    chainerx::Shape to = shape;
    int64_t known = 1;
    int wildcard = -1;
    for (int i = 0; i < static_cast<int>(to.size()); ++i) {
        if (to[i] == 0) {
            CHECK_LT(i, data.ndim());
            to[i] = data.shape()[i];
        }
        if (to[i] == -1) {
            CHECK_EQ(-1, wildcard) << "more than one -1 in a Reshape";
            wildcard = i;
        } else {
            known *= to[i];
        }
    }
    if (wildcard >= 0) to[wildcard] = known ? data.GetTotalSize() / known : 0;
    CHECK_EQ(data.GetTotalSize(), to.GetTotalSize()) << "Reshape changes the number of elements";
    return AsContiguous(data).Reshape(to);  // chainerx::Reshape copies likewise when the strides do not allow a view
}

}  // namespace runtime
}  // namespace chainer_compiler
