// FixedBatchNormalizationOp (runtime/ops/normalization.cc:210-225 of the chainer-compiler tree) on the hip
// backend: the inference form of BatchNormalization, which the quantizer leaves in float behind an integer
// convolution; and SoftmaxOp (runtime/ops/activation.cc:93-95).  The arithmetic is in chx_hip_fixed_batch_norm_f32
// and chx_hip_softmax_f32.
#include "../gen/gen_chxvm_ops.h"

namespace chainer_compiler {
namespace runtime {

chainerx::Array AsContiguous(const chainerx::Array& a);

chainerx::Array FixedBatchNormalizationOp::RunImpl(
        ChxVMState* st, const chainerx::Array& x, const chainerx::Array& s, const chainerx::Array& bias, const chainerx::Array& mean,
        const chainerx::Array& var) {
    CHECK(x.dtype() == chainerx::Dtype::kFloat32) << "FixedBatchNormalization: x must be float32 on the hip backend, not " << x.dtype();
    CHECK_LE(2, x.ndim()) << "FixedBatchNormalization: x needs a batch and a channel axis";
    const chainerx::Array sd = AsContiguous(s), bd = AsContiguous(bias), md = AsContiguous(mean), vd = AsContiguous(var);
    // the result in the layout of x when x is a channels-last view, dense otherwise
    const bool channels_last = x.ndim() == 4 && x.shape()[1] > 1 && x.strides()[1] == 4 && !x.IsContiguous();
    chainerx::Array y = channels_last ? chainerx::EmptyChannelsLast(x.shape(), chainerx::Dtype::kFloat32)
                                      : chainerx::Empty(x.shape(), chainerx::Dtype::kFloat32);
    chx_hip_tensor xt = x.hip(), st_ = sd.hip(), bt = bd.hip(), mt = md.hip(), vt = vd.hip(), yt = y.hip();
    CHXVM_HIP_CALL(chx_hip_fixed_batch_norm_f32(&xt, &st_, &bt, &mt, &vt, static_cast<float>(epsilon), &yt, chainerx::CurrentStream()));
    return y;
}

// SoftmaxOp::RunImpl, runtime/ops/activation.cc:93-95 (RunSoftmax :66-89): the classifier head's last node.
chainerx::Array SoftmaxOp::RunImpl(ChxVMState* st, const chainerx::Array& input) {
    CHECK(input.dtype() == chainerx::Dtype::kFloat32) << "Softmax: float32 only on the hip backend, not " << input.dtype();
    int ax = static_cast<int>(axis);
    if (ax < 0) ax += input.ndim();
    CHECK_LE(0, ax);
    CHECK_GT(input.ndim(), ax);
    const chainerx::Array x = AsContiguous(input);
    chainerx::Array y = chainerx::Empty(x.shape(), chainerx::Dtype::kFloat32);
    chx_hip_tensor xt = x.hip(), yt = y.hip();
    CHXVM_HIP_CALL(chx_hip_softmax_f32(&xt, ax, is_onnx_semantics ? 1 : 0, &yt, chainerx::CurrentStream()));
    return y;
}

}  // namespace runtime
}  // namespace chainer_compiler
