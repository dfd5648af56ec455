// RunImpl bodies of the quantized ops on the hip backend: the signatures of
// runtime/ops/quantize.cc:48-146 of the chainer-compiler tree, each body a shape inference, an
// output allocation and one call into the C ABI (include/chx_hip.h).
#include "../chainerx_util.h"
#include "../gen/gen_chxvm_ops.h"
#include "../chxvm.h"

#include <atomic>

namespace chainer_compiler {
namespace runtime {

namespace {

std::atomic<int64_t> g_residual_fusions{0};

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
                &xt, static_cast<float>(x_scale), static_cast<int32_t>(static_cast<int64_t>(x_zero_point)), &wt, &st2, &zt,
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
                &xt, static_cast<float>(x_scale), static_cast<int32_t>(static_cast<int64_t>(x_zero_point)), &wt, &st2, &zt,
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
            chainerx::Array out = chainerx::EmptyChannelsLastPadded(y_shape, req->out_dtype);
            chx_hip_tensor xt = q_x.hip(), rt = req->r.hip(), ot = out.hip();
            const int rc = chx_hip_qconv_plan_run_add(
                    impl_->plan, &xt, static_cast<float>(x_scale), static_cast<int32_t>(static_cast<int64_t>(x_zero_point)),
                    req->y_scale, req->y_zero_point, static_cast<int32_t>(req->y_dtype), flags, &rt, req->r_scale, req->r_zero_point,
                    req->out_scale, req->out_zero_point, req->relu ? 1 : 0, &ot, chainerx::CurrentStream());
            if (rc == CHX_HIP_OK) {
                req->out = out;
                req->done = true;
                ++g_residual_fusions;
                st->count_residual_fusion();
                return chainerx::Array();
            }
            CHECK_EQ(CHX_HIP_EUNSUPPORTED, rc) << chx_hip_last_error();  // unsupported: run the ops one by one
        }
    }
    // 8-bit activations leave a convolution channels-last, whatever layout came in
    chainerx::Array y = chainerx::EmptyChannelsLastPadded(y_shape, y_zero_point.dtype());
    chx_hip_tensor xt = q_x.hip(), yt = y.hip();
    CHXVM_HIP_CALL(chx_hip_qconv_plan_run(
            impl_->plan, &xt, static_cast<float>(x_scale), static_cast<int32_t>(static_cast<int64_t>(x_zero_point)),
            static_cast<float>(y_scale), static_cast<int32_t>(static_cast<int64_t>(y_zero_point)), flags, &yt, chainerx::CurrentStream()));
    return y;
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
