// RunImpl bodies of the quantized ops on the hip backend: the signatures of
// runtime/ops/quantize.cc:48-146 of the chainer-compiler tree, each body a shape inference, an
// output allocation and one call into the C ABI (include/chx_hip.h).
#include "../chainerx_util.h"
#include "../gen/gen_chxvm_ops.h"
#include "../chxvm.h"

#include <atomic>
#include <iostream>

namespace chainer_compiler {
namespace runtime {

namespace {

std::atomic<int64_t> g_residual_fusions{0};
std::atomic<int64_t> g_minus_128_stores{0};

// A uint8 value kept as code - 128 in an int8 array: what a producer leaves in a variable for which
// ChxVMState::store_minus_128 holds.  Such an array is an int8 tensor with the zero point lowered by 128.
bool HoldsCodesMinus128(ChxVMState* st, int slot, const chainerx::Array& a, chainerx::Dtype type_in_program) {
    return st->store_minus_128(slot) && a.dtype() == chainerx::Dtype::kInt8 && type_in_program == chainerx::Dtype::kUInt8;
}

StrictScalar DefaultZeroPoint() {
    // an absent zero point is uint8 0 (runtime/ops/quantize.cc:50-51,57-58)
    return StrictScalar(chainerx::Dtype::kUInt8, chainerx::Scalar(0u), false);
}

void CheckQuantizedDtype(chainerx::Dtype dt, const char* what) {
    CHECK(dt == chainerx::Dtype::kUInt8 || dt == chainerx::Dtype::kInt8) << what << " must be uint8 or int8, got " << dt;
}

// outputs follow the input's layout: channels-last in, channels-last out
chainerx::Array EmptyLike4d(const chainerx::Array& x, const chainerx::Shape& shape, chainerx::Dtype dtype) {
    const bool channels_last = x.ndim() == 4 && !x.IsContiguous() && x.strides()[1] == x.GetItemSize();
    return channels_last ? chainerx::EmptyChannelsLast(shape, dtype) : chainerx::Empty(shape, dtype);
}

}  // namespace

int64_t QLinearConvResidualFusions() {
    return g_residual_fusions.load();
}

int64_t Minus128Stores() {
    return g_minus_128_stores.load();
}

chainerx::Array PlainCodes(const chainerx::Array& minus_128) {
    CHECK(minus_128.dtype() == chainerx::Dtype::kInt8);
    const bool channels_last = minus_128.ndim() == 4 && !minus_128.IsContiguous() && minus_128.strides()[1] == minus_128.GetItemSize();
    chainerx::Array plain = channels_last ? chainerx::EmptyChannelsLastPadded(minus_128.shape(), chainerx::Dtype::kUInt8)
                                          : chainerx::Empty(minus_128.shape(), chainerx::Dtype::kUInt8);
    chx_hip_tensor xt = minus_128.hip(), yt = plain.hip();
    CHXVM_HIP_CALL(chx_hip_codes_minus_128(&xt, &yt, chainerx::CurrentStream()));
    return plain;
}

chainerx::Array QuantizeLinearOp::RunImpl(
        ChxVMState* st, const chainerx::Array& x, const StrictScalar& y_scale, const absl::optional<StrictScalar>& y_zero_point_opt) {
    const StrictScalar y_zero_point = y_zero_point_opt.has_value() ? *y_zero_point_opt : DefaultZeroPoint();
    CheckQuantizedDtype(y_zero_point.dtype(), "QuantizeLinear zero point");  // CHECK_EQ(kUInt8, ...), quantize.cc:24
    chainerx::Array y = EmptyLike4d(x, x.shape(), y_zero_point.dtype());
    chx_hip_tensor xt = x.hip(), yt = y.hip();
    CHXVM_HIP_CALL(chx_hip_quantize_linear(&xt, static_cast<float>(y_scale), static_cast<int32_t>(static_cast<int64_t>(y_zero_point)),
                                           CHX_HIP_ROUND_REFERENCE, &yt, chainerx::CurrentStream()));
    return y;
}

chainerx::Array DequantizeLinearOp::RunImpl(
        ChxVMState* st, const chainerx::Array& x, const StrictScalar& x_scale, const absl::optional<StrictScalar>& x_zero_point_opt) {
    const StrictScalar x_zero_point = x_zero_point_opt.has_value() ? *x_zero_point_opt : DefaultZeroPoint();
    chainerx::Array y = EmptyLike4d(x, x.shape(), chainerx::Dtype::kFloat32);
    chx_hip_tensor xt = x.hip(), yt = y.hip();
    CHXVM_HIP_CALL(chx_hip_dequantize_linear(&xt, static_cast<float>(x_scale),
                                             static_cast<int32_t>(static_cast<int64_t>(x_zero_point)), &yt, chainerx::CurrentStream()));
    return y;
}

// Per-instruction state: the plan holds the weights repacked for the MFMA kernel (and the device addresses
// of the scales, zero points and bias).  The reference re-dequantizes the weights on every call
// (quantize.cc:76-88); an op object lives as long as the program, so for operands that are constants of
// the program the repacking is done once.  The plan is tied to the four operand arrays it was built
// from: the op keeps a reference to each (their memory cannot be released and handed out again while the
// plan lives) and rebuilds the plan when a run brings other ones.  Operands that come from the caller
// of the runtime (program inputs: memory that may be rewritten or released between runs) get no plan;
// such a convolution goes through the one-shot entry point, which repacks per call.
class QLinearConvOp::QLinearConvImpl {
public:
    chx_hip_qconv_plan* plan = nullptr;
    chx_hip_conv_params params;
    chainerx::Array w, w_scale, w_zero_point, bias;  // what the plan was built from
    bool minus_128_refused = false;  // the kernel that runs this plan does not write the minus-128 storage

    bool Matches(const chainerx::Array& q_w, const chainerx::Array& s, const chainerx::Array& z, const absl::optional<chainerx::Array>& b,
                 const chx_hip_conv_params& p) const {
        auto same = [](const chainerx::Array& kept, const chainerx::Array& now) {
            return !kept.IsNullHandle() && kept.raw_data() == now.raw_data() && kept.offset() == now.offset() &&
                   kept.shape() == now.shape() && kept.strides() == now.strides() && kept.dtype() == now.dtype();
        };
        if (!same(w, q_w) || !same(w_scale, s) || !same(w_zero_point, z)) return false;
        if (b.has_value() != !bias.IsNullHandle()) return false;
        if (b.has_value() && !same(bias, *b)) return false;
        return memcmp(&params, &p, sizeof(p)) == 0;
    }
    void Drop() {
        chx_hip_qconv_plan_destroy(plan);
        plan = nullptr;
        w = w_scale = w_zero_point = bias = chainerx::Array();
        minus_128_refused = false;
    }
};

void QLinearConvOp::InitImpl() {
    impl_ = new QLinearConvImpl();
}

QLinearConvOp::~QLinearConvOp() {
    if (impl_) chx_hip_qconv_plan_destroy(impl_->plan);
    delete impl_;
}

chainerx::Array QLinearConvOp::RunImpl(
        ChxVMState* st,
        const chainerx::Array& q_x,
        const StrictScalar& x_scale,
        const StrictScalar& x_zero_point,
        const chainerx::Array& q_w,
        const chainerx::Array& w_scale,
        const chainerx::Array& w_zero_point,
        const StrictScalar& y_scale,
        const StrictScalar& y_zero_point,
        const absl::optional<chainerx::Array>& b) {
    CHECK_EQ(w_scale.GetTotalSize(), w_zero_point.GetTotalSize());
    CHECK_EQ(w_scale.shape().size(), w_zero_point.shape().size());
    CheckQuantizedDtype(y_zero_point.dtype(), "QLinearConv y_zero_point");
    // (an input kept as code - 128 is an int8 tensor with the zero point 128 lower: every kernel takes it as that)
    const int32_t x_zp = static_cast<int32_t>(static_cast<int64_t>(x_zero_point)) - (HoldsCodesMinus128(st, this->x, q_x, x_zero_point.dtype()) ? 128 : 0);
    if (q_x.ndim() != 4) {
        // one or three spatial axes: the rank-generic entry point, operands as they are, a dense result
        chainerx::Shape nd_shape;
        const chx_hip_conv_nd_params np = MakeConvNdParams(q_x, q_w, strides, pads, group, auto_pad, &nd_shape);
        const uint32_t nd_flags =
                CHX_HIP_ROUND_REFERENCE | (st->options().qlinearconv_onnx_int32_bias ? CHX_HIP_BIAS_ONNX_INT32 : CHX_HIP_BIAS_REFERENCE_FLOAT);
        chainerx::Array y = chainerx::Empty(nd_shape, y_zero_point.dtype());
        chx_hip_tensor xt = q_x.hip(), wt = q_w.hip(), st2 = w_scale.hip(), zt = w_zero_point.hip(), yt = y.hip(), bt;
        if (b.has_value()) bt = b->hip();
        CHXVM_HIP_CALL(chx_hip_qlinear_conv_nd(
                &xt, static_cast<float>(x_scale), x_zp, &wt, &st2, &zt,
                static_cast<float>(y_scale), static_cast<int32_t>(static_cast<int64_t>(y_zero_point)), b.has_value() ? &bt : nullptr, &np,
                nd_flags, &yt, chainerx::CurrentStream()));
        return y;
    }
    const chx_hip_conv_params p = MakeConvParams(q_x, q_w, strides, pads, group, auto_pad);
    const chainerx::Shape y_shape = ConvOutputShape(q_x, q_w, p);
    // The reference adds the bias as an unscaled float after the convolution (runtime/ops/quantize.cc:93);
    // networks quantized for the ONNX operator carry an int32 bias at scale x_scale * w_scale[oc].  The
    // options of the run say which of the two this program means.
    const uint32_t flags =
            CHX_HIP_ROUND_REFERENCE | (st->options().qlinearconv_onnx_int32_bias ? CHX_HIP_BIAS_ONNX_INT32 : CHX_HIP_BIAS_REFERENCE_FLOAT);
    const bool constants = !q_w.IsBorrowed() && !w_scale.IsBorrowed() && !w_zero_point.IsBorrowed() && !(b.has_value() && b->IsBorrowed());
    if (!constants) {
        if (impl_->plan) impl_->Drop();
        chainerx::Array y = chainerx::EmptyChannelsLastPadded(y_shape, y_zero_point.dtype());
        chx_hip_tensor xt = q_x.hip(), wt = q_w.hip(), st2 = w_scale.hip(), zt = w_zero_point.hip(), yt = y.hip(), bt;
        if (b.has_value()) bt = b->hip();
        CHXVM_HIP_CALL(chx_hip_qlinear_conv(
                &xt, static_cast<float>(x_scale), x_zp, &wt, &st2, &zt,
                static_cast<float>(y_scale), static_cast<int32_t>(static_cast<int64_t>(y_zero_point)), b.has_value() ? &bt : nullptr, &p,
                flags, &yt, chainerx::CurrentStream()));
        return y;
    }
    if (impl_->plan && !impl_->Matches(q_w, w_scale, w_zero_point, b, p)) impl_->Drop();
    if (!impl_->plan) {
        chx_hip_tensor wt = q_w.hip(), st2 = w_scale.hip(), zt = w_zero_point.hip(), bt;
        if (b.has_value()) bt = b->hip();
        CHXVM_HIP_CALL(chx_hip_qconv_plan_create(&wt, &st2, &zt, b.has_value() ? &bt : nullptr, &p, nullptr, &impl_->plan));
        impl_->params = p;
        impl_->w = q_w;
        impl_->w_scale = w_scale;
        impl_->w_zero_point = w_zero_point;
        impl_->bias = b.has_value() ? *b : chainerx::Array();
    }
    if (std::vector<chx_hip_qconv_plan*>* pinned = st->options().pinned_plans) {
        // this run is being recorded: the recording holds addresses inside the plan
        CHXVM_HIP_CALL(chx_hip_qconv_plan_pin(impl_->plan, 1));
        pinned->push_back(impl_->plan);
    }
    if (QLinearConvResidualRequest* req = st->residual_request()) {
        const bool same_quantization = static_cast<float>(y_scale) == req->y_scale &&
                                       static_cast<int64_t>(y_zero_point) == req->y_zero_point && y_zero_point.dtype() == req->y_dtype;
        if (same_quantization && !req->r.IsNullHandle() && req->r.shape() == y_shape) {
            // the sum in the minus-128 storage where its variable allows it; the kernel's refusal of that storage
            // (remembered) is not a refusal of the sum
            const bool minus_128 = st->store_minus_128(req->out_slot) && req->out_dtype == chainerx::Dtype::kUInt8 && !impl_->minus_128_refused;
            for (int attempt = minus_128 ? 0 : 1; attempt < 2; ++attempt) {
                const bool signed_storage = attempt == 0;
                chainerx::Array out = chainerx::EmptyChannelsLastPadded(y_shape, signed_storage ? chainerx::Dtype::kInt8 : req->out_dtype);
                chx_hip_tensor xt = q_x.hip(), rt = req->r.hip(), ot = out.hip();
                const int rc = chx_hip_qconv_plan_run_add(
                        impl_->plan, &xt, static_cast<float>(x_scale), x_zp, req->y_scale, req->y_zero_point, static_cast<int32_t>(req->y_dtype),
                        flags | (signed_storage ? CHX_HIP_STORE_MINUS_128 : 0u), &rt, req->r_scale, req->r_zero_point, req->out_scale,
                        req->out_zero_point, req->relu ? 1 : 0, &ot, chainerx::CurrentStream());
                if (rc == CHX_HIP_OK) {
                    req->out = out;
                    req->done = true;
                    ++g_residual_fusions;
                    if (signed_storage) ++g_minus_128_stores;
                    st->count_residual_fusion();
                    return chainerx::Array();
                }
                CHECK_EQ(CHX_HIP_EUNSUPPORTED, rc) << chx_hip_last_error();  // unsupported: run the ops one by one
                if (signed_storage) impl_->minus_128_refused = true;
            }
        }
    }
    // 8-bit activations leave a convolution channels-last, whatever layout came in
    if (st->store_minus_128(this->y) && y_zero_point.dtype() == chainerx::Dtype::kUInt8 && !impl_->minus_128_refused) {
        chainerx::Array y_minus_128 = chainerx::EmptyChannelsLastPadded(y_shape, chainerx::Dtype::kInt8);
        chx_hip_tensor xt = q_x.hip(), yt = y_minus_128.hip();
        const int rc = chx_hip_qconv_plan_run(
                impl_->plan, &xt, static_cast<float>(x_scale), x_zp, static_cast<float>(y_scale),
                static_cast<int32_t>(static_cast<int64_t>(y_zero_point)), flags | CHX_HIP_STORE_MINUS_128, &yt, chainerx::CurrentStream());
        if (rc == CHX_HIP_OK) {
            ++g_minus_128_stores;
            return y_minus_128;
        }
        CHECK_EQ(CHX_HIP_EUNSUPPORTED, rc) << chx_hip_last_error();  // a kernel that writes plain codes only
        impl_->minus_128_refused = true;
    }
    chainerx::Array y = chainerx::EmptyChannelsLastPadded(y_shape, y_zero_point.dtype());
    chx_hip_tensor xt = q_x.hip(), yt = y.hip();
    CHXVM_HIP_CALL(chx_hip_qconv_plan_run(
            impl_->plan, &xt, static_cast<float>(x_scale), x_zp, static_cast<float>(y_scale),
            static_cast<int32_t>(static_cast<int64_t>(y_zero_point)), flags, &yt, chainerx::CurrentStream()));
    return y;
}

namespace {

std::atomic<int64_t> g_pair_fusions{0};

// b appended to a along the first axis, dense
chainerx::Array ConcatFirstAxis(const chainerx::Array& a, const chainerx::Array& b) {
    chainerx::Shape shape = a.shape();
    shape[0] += b.shape()[0];
    chainerx::Array y = chainerx::Empty(shape, a.dtype());
    const chainerx::Array* parts[2] = {&a, &b};
    int64_t at = 0;
    for (const chainerx::Array* part : parts) {
        const chainerx::Array span = y.Narrow(0, at, part->shape()[0]);
        chx_hip_tensor xt = part->hip(), yt = span.hip();
        CHXVM_HIP_CALL(chx_hip_cast(&xt, &yt, chainerx::CurrentStream()));  // same element type on both sides: a copy
        at += part->shape()[0];
    }
    return y;
}

// The variable slots and attributes of a QLinearConv instruction (the op class keeps its own private).
struct QLinearConvSlots {
    explicit QLinearConvSlots(const ChxVMInstructionProto& inst)
        : x(inst.inputs[0].array), x_scale(inst.inputs[1].scalar), x_zero_point(inst.inputs[2].scalar), w(inst.inputs[3].array),
          w_scale(inst.inputs[4].array), w_zero_point(inst.inputs[5].array), y_scale(inst.inputs[6].scalar),
          y_zero_point(inst.inputs[7].scalar), b(inst.inputs[8].array), strides(inst.inputs[9].ints.begin(), inst.inputs[9].ints.end()),
          pads(inst.inputs[10].ints.begin(), inst.inputs[10].ints.end()), group(static_cast<int>(inst.inputs[11].i)),
          auto_pad(inst.inputs[12].s), y(inst.outputs[0]) {
    }
    int x, x_scale, x_zero_point, w, w_scale, w_zero_point, y_scale, y_zero_point, b;
    chainerx::StackVector<int64_t, chainerx::kMaxNdim> strides, pads;
    int group;
    std::string auto_pad;
    int y;
};

class QLinearConvPairOp : public ChxVMOp {
public:
    QLinearConvPairOp(const ChxVMInstructionProto& first, const ChxVMInstructionProto& second)
        : ChxVMOp(first), first_(new QLinearConvOp(first)), second_(new QLinearConvOp(second)), a_(new QLinearConvSlots(first)),
          b_(new QLinearConvSlots(second)) {
    }
    ~QLinearConvPairOp() override {
        chx_hip_qconv_plan_destroy(plan_);
    }
    void InitImpl() override {
        first_->InitImpl();
        second_->InitImpl();
    }
    void Run(ChxVMState* st) override {
        if (!RunAsOne(st)) {
            first_->Run(st);
            second_->Run(st);
        }
    }

private:
    struct Operands {
        chainerx::Array w, w_scale, w_zero_point;
        absl::optional<chainerx::Array> bias;
    };
    static bool Same(const chainerx::Array& kept, const chainerx::Array& now) {
        return !kept.IsNullHandle() && kept.raw_data() == now.raw_data() && kept.offset() == now.offset() && kept.shape() == now.shape() &&
               kept.strides() == now.strides() && kept.dtype() == now.dtype();
    }
    static bool Same(const Operands& kept, const Operands& now) {
        if (!Same(kept.w, now.w) || !Same(kept.w_scale, now.w_scale) || !Same(kept.w_zero_point, now.w_zero_point)) return false;
        if (kept.bias.has_value() != now.bias.has_value()) return false;
        return !kept.bias.has_value() || Same(*kept.bias, *now.bias);
    }
    static bool Constants(const Operands& o) {
        return !o.w.IsBorrowed() && !o.w_scale.IsBorrowed() && !o.w_zero_point.IsBorrowed() && !(o.bias.has_value() && o.bias->IsBorrowed());
    }
    static Operands Fetch(ChxVMState* st, const QLinearConvSlots& op) {
        return Operands{st->GetArray(op.w), st->GetArray(op.w_scale), st->GetArray(op.w_zero_point), st->GetOptionalArray(op.b)};
    }

    // false: the two instructions have to run on their own (nothing has been written)
    bool RunAsOne(ChxVMState* st) {
        for (const QLinearConvSlots* op : {a_.get(), b_.get()})
            for (int slot : {op->x, op->w, op->w_scale, op->w_zero_point})
                if (slot < 0 || st->GetVar(slot)->IsNull()) return false;
        const chainerx::Array x = st->GetArray(a_->x);
        const Operands oa = Fetch(st, *a_), ob = Fetch(st, *b_);
        const StrictScalar x_scale = st->GetScalar(a_->x_scale), x_zero_point = st->GetScalar(a_->x_zero_point);
        const StrictScalar y1_scale = st->GetScalar(a_->y_scale), y1_zero_point = st->GetScalar(a_->y_zero_point);
        const StrictScalar y2_scale = st->GetScalar(b_->y_scale), y2_zero_point = st->GetScalar(b_->y_zero_point);
        // the same activation quantization on both (they read the same value: anything else would be a program that
        // interprets one tensor in two ways), per-channel weight scales, weights that are constants of the program
        if (static_cast<float>(x_scale) != static_cast<float>(st->GetScalar(b_->x_scale)) ||
            static_cast<int64_t>(x_zero_point) != static_cast<int64_t>(st->GetScalar(b_->x_zero_point)))
            return false;
        if (x.ndim() != 4 || oa.w.ndim() != 4 || ob.w.ndim() != 4 || oa.w.dtype() != ob.w.dtype() || !Constants(oa) || !Constants(ob)) return false;
        for (int d = 1; d < 4; ++d)
            if (oa.w.shape()[d] != ob.w.shape()[d]) return false;
        const int64_t oc1 = oa.w.shape()[0], oc2 = ob.w.shape()[0];
        auto per_channel = [](const Operands& o, int64_t oc) {
            return o.w_scale.ndim() == 1 && o.w_scale.shape()[0] == oc && o.w_zero_point.ndim() == 1 && o.w_zero_point.shape()[0] == oc &&
                   (!o.bias.has_value() || (o.bias->ndim() == 1 && o.bias->shape()[0] == oc));
        };
        if (oc1 % 64 != 0 || !per_channel(oa, oc1) || !per_channel(ob, oc2) || oa.bias.has_value() != ob.bias.has_value()) return false;
        if (oa.w_zero_point.dtype() != ob.w_zero_point.dtype() || oa.w_scale.dtype() != ob.w_scale.dtype()) return false;
        const bool is_q8 = (y1_zero_point.dtype() == chainerx::Dtype::kUInt8 || y1_zero_point.dtype() == chainerx::Dtype::kInt8) &&
                           (y2_zero_point.dtype() == chainerx::Dtype::kUInt8 || y2_zero_point.dtype() == chainerx::Dtype::kInt8);
        if (!is_q8) return false;
        const chx_hip_conv_params p = MakeConvParams(x, oa.w, a_->strides, a_->pads, a_->group, a_->auto_pad);
        const chx_hip_conv_params p2 = MakeConvParams(x, ob.w, b_->strides, b_->pads, b_->group, b_->auto_pad);
        if (memcmp(&p, &p2, sizeof(p)) != 0 || p.group != 1) return false;
        if (plan_ && !(Same(kept_a_, oa) && Same(kept_b_, ob) && memcmp(&p, &params_, sizeof(p)) == 0)) {
            chx_hip_qconv_plan_destroy(plan_);
            plan_ = nullptr;
        }
        if (!plan_) {
            if (failed_ && Same(kept_a_, oa) && Same(kept_b_, ob)) return false;  // these operands were refused before
            w_ = ConcatFirstAxis(oa.w, ob.w);
            w_scale_ = ConcatFirstAxis(oa.w_scale, ob.w_scale);
            w_zero_point_ = ConcatFirstAxis(oa.w_zero_point, ob.w_zero_point);
            bias_ = oa.bias.has_value() ? ConcatFirstAxis(*oa.bias, *ob.bias) : chainerx::Array();
            chx_hip_tensor wt = w_.hip(), st2 = w_scale_.hip(), zt = w_zero_point_.hip(), bt;
            if (oa.bias.has_value()) bt = bias_.hip();
            CHXVM_HIP_CALL(chx_hip_qconv_plan_create(&wt, &st2, &zt, oa.bias.has_value() ? &bt : nullptr, &p, nullptr, &plan_));
            params_ = p;
            kept_a_ = oa;
            kept_b_ = ob;
            failed_ = false;
        }
        const uint32_t flags =
                CHX_HIP_ROUND_REFERENCE | (st->options().qlinearconv_onnx_int32_bias ? CHX_HIP_BIAS_ONNX_INT32 : CHX_HIP_BIAS_REFERENCE_FLOAT);
        chainerx::Shape y1_shape = ConvOutputShape(x, oa.w, p), y2_shape = ConvOutputShape(x, ob.w, p);
        const int32_t x_zp = static_cast<int32_t>(static_cast<int64_t>(x_zero_point)) - (HoldsCodesMinus128(st, a_->x, x, x_zero_point.dtype()) ? 128 : 0);
        // each result in the minus-128 storage where its variable allows it
        const bool s1 = st->store_minus_128(a_->y) && y1_zero_point.dtype() == chainerx::Dtype::kUInt8;
        const bool s2 = st->store_minus_128(b_->y) && y2_zero_point.dtype() == chainerx::Dtype::kUInt8;
        chainerx::Array y1 = chainerx::EmptyChannelsLastPadded(y1_shape, s1 ? chainerx::Dtype::kInt8 : y1_zero_point.dtype());
        chainerx::Array y2 = chainerx::EmptyChannelsLastPadded(y2_shape, s2 ? chainerx::Dtype::kInt8 : y2_zero_point.dtype());
        chx_hip_tensor xt = x.hip(), y1t = y1.hip(), y2t = y2.hip();
        const int rc = chx_hip_qconv_plan_run_pair(
                plan_, &xt, static_cast<float>(x_scale), x_zp, static_cast<int32_t>(oc1), static_cast<float>(y1_scale),
                static_cast<int32_t>(static_cast<int64_t>(y1_zero_point)), flags | (s1 ? CHX_HIP_STORE_MINUS_128 : 0u), &y1t,
                static_cast<float>(y2_scale), static_cast<int32_t>(static_cast<int64_t>(y2_zero_point)),
                flags | (s2 ? CHX_HIP_STORE_MINUS_128 : 0u), &y2t, chainerx::CurrentStream());
        if (rc == CHX_HIP_OK) g_minus_128_stores += (s1 ? 1 : 0) + (s2 ? 1 : 0);
        if (rc == CHX_HIP_EUNSUPPORTED) {
            // layouts or weights the one-launch kernel does not take: remembered, so that the weights are not joined again
            chx_hip_qconv_plan_destroy(plan_);
            plan_ = nullptr;
            failed_ = true;
            return false;
        }
        CHECK_EQ(CHX_HIP_OK, rc) << chx_hip_last_error();
        if (std::vector<chx_hip_qconv_plan*>* pinned = st->options().pinned_plans) {
            // this run is being recorded: the recording holds addresses inside the plan
            CHXVM_HIP_CALL(chx_hip_qconv_plan_pin(plan_, 1));
            pinned->push_back(plan_);
        }
        if (st->trace_level())
            std::cerr << "$" << a_->y << ", $" << b_->y << " = QLinearConv x 2 in one launch($" << a_->x << ")" << std::endl;
        st->SetArray(a_->y, y1);
        st->SetArray(b_->y, y2);
        ++g_pair_fusions;
        return true;
    }

    std::unique_ptr<QLinearConvOp> first_, second_;  // the instructions as they are, for operands the one launch does not take
    std::unique_ptr<QLinearConvSlots> a_, b_;
    chx_hip_qconv_plan* plan_ = nullptr;
    chx_hip_conv_params params_;
    Operands kept_a_, kept_b_;               // what the plan was built from
    chainerx::Array w_, w_scale_, w_zero_point_, bias_;  // the joined operands the plan points into
    bool failed_ = false;
};

}  // namespace

std::unique_ptr<ChxVMOp> MakeQLinearConvPairOp(const ChxVMInstructionProto& first, const ChxVMInstructionProto& second) {
    return std::unique_ptr<ChxVMOp>(new QLinearConvPairOp(first, second));
}

int64_t QLinearConvPairFusions() {
    return g_pair_fusions.load();
}

chainerx::Array MatMulIntegerOp::RunImpl(
        ChxVMState* st,
        const chainerx::Array& q_a,
        const chainerx::Array& q_b,
        const absl::optional<chainerx::Array>& a_zero_point,
        const absl::optional<chainerx::Array>& b_zero_point) {
    if (a_zero_point.has_value()) CHECK_GE(1, a_zero_point->shape().size());
    if (b_zero_point.has_value()) CHECK_GE(1, b_zero_point->shape().size());
    CHECK_LE(2, q_a.ndim());
    CHECK_EQ(q_a.ndim(), q_b.ndim()) << "MatMulInteger operands must have the same rank on the hip backend";
    chainerx::Shape shape(q_a.shape().begin(), q_a.shape().end() - 1);
    shape.push_back(q_b.shape()[q_b.ndim() - 1]);
    chainerx::Array y = chainerx::Empty(shape, chainerx::Dtype::kInt32);
    chx_hip_tensor at = q_a.hip(), bt = q_b.hip(), yt = y.hip(), azt, bzt;
    if (a_zero_point.has_value()) azt = a_zero_point->hip();
    if (b_zero_point.has_value()) bzt = b_zero_point->hip();
    CHXVM_HIP_CALL(chx_hip_matmul_integer(&at, &bt, a_zero_point.has_value() ? &azt : nullptr,
                                          b_zero_point.has_value() ? &bzt : nullptr, &yt, chainerx::CurrentStream()));
    return y;
}

chainerx::Array ConvIntegerOp::RunImpl(
        ChxVMState* st,
        const chainerx::Array& q_x,
        const chainerx::Array& q_w,
        const absl::optional<StrictScalar>& x_zero_point,
        const absl::optional<chainerx::Array>& w_zero_point_opt) {
    if (q_x.ndim() != 4) {
        chainerx::Shape nd_shape;
        const chx_hip_conv_nd_params np = MakeConvNdParams(q_x, q_w, strides, pads, group, auto_pad, &nd_shape);
        chainerx::Array y = chainerx::Empty(nd_shape, chainerx::Dtype::kInt32);
        chx_hip_tensor xt = q_x.hip(), wt = q_w.hip(), yt = y.hip(), zt;
        if (w_zero_point_opt.has_value()) zt = w_zero_point_opt->hip();
        const int32_t xz = x_zero_point.has_value() ? static_cast<int32_t>(static_cast<int64_t>(*x_zero_point)) : 0;
        CHXVM_HIP_CALL(chx_hip_conv_integer_nd(&xt, &wt, xz, w_zero_point_opt.has_value() ? &zt : nullptr, &np, &yt, chainerx::CurrentStream()));
        return y;
    }
    const chx_hip_conv_params p = MakeConvParams(q_x, q_w, strides, pads, group, auto_pad);
    chainerx::Array y = EmptyLike4d(q_x, ConvOutputShape(q_x, q_w, p), chainerx::Dtype::kInt32);
    chx_hip_tensor xt = q_x.hip(), wt = q_w.hip(), yt = y.hip(), zt;
    if (w_zero_point_opt.has_value()) zt = w_zero_point_opt->hip();
    const int32_t xz = x_zero_point.has_value() ? static_cast<int32_t>(static_cast<int64_t>(*x_zero_point)) : 0;
    CHXVM_HIP_CALL(chx_hip_conv_integer(&xt, &wt, xz, w_zero_point_opt.has_value() ? &zt : nullptr, &p, &yt, chainerx::CurrentStream()));
    return y;
}

// MatMulOp::RunImpl, runtime/ops/math.cc:156-158 (NumpyMatMul, runtime/chainerx_util.cc:210-230) for
// matrices.  Between two DequantizeLinear and one QuantizeLinear (the sequence ReplaceQLinearMatMul
// leaves, compiler/simplifier.cc:675-694) ChxVM fuses the product into one quantized kernel when it
// loads the program (chxvm.cc) and this op does not run; anywhere else it is a float32 product.
chainerx::Array MatMulOp::RunImpl(ChxVMState* st, const chainerx::Array& a, const chainerx::Array& b) {
    CHECK(a.ndim() == 2 && b.ndim() == 2) << "float MatMul of operands that are not matrices is not computed on the hip backend";
    CHECK(a.dtype() == chainerx::Dtype::kFloat32 && b.dtype() == chainerx::Dtype::kFloat32) << "float MatMul: float32 operands only";
    chainerx::Array y = chainerx::Empty(chainerx::Shape{a.shape()[0], b.shape()[1]}, chainerx::Dtype::kFloat32);
    chx_hip_tensor at = a.hip(), bt = b.hip(), yt = y.hip();
    CHXVM_HIP_CALL(chx_hip_gemm_f32(&at, &bt, nullptr, 1.f, 1.f, 0, 0, &yt, chainerx::CurrentStream()));
    return y;
}

}  // namespace runtime
}  // namespace chainer_compiler
