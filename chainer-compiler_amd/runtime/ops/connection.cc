// The float layers around a quantized network on the hip backend: ConvOp (runtime/ops/connection.cc:24-30), GemmOp and MatMulOp
// (runtime/ops/math.cc:156-177 of the chainer-compiler tree), LinearOp (runtime/ops/connection.cc:12-15),
// FlattenOp (runtime/ops/manipulation.cc:20-28).  The products run in chx_hip_gemm_f32 /
// chx_hip_linear_f32; Flatten is a view, after a device copy when the array is not dense.
#include "../chainerx_util.h"
#include "../gen/gen_chxvm_ops.h"

namespace chainer_compiler {
namespace runtime {

namespace {

void CheckFloat32(const chainerx::Array& a, const char* op, const char* name) {
    CHECK(a.dtype() == chainerx::Dtype::kFloat32) << op << ": " << name << " must be float32 on the hip backend, not " << a.dtype();
}

// outputs follow the input's layout: channels-last in, channels-last out
chainerx::Array EmptyLike4d(const chainerx::Array& x, const chainerx::Shape& shape, chainerx::Dtype dtype) {
    const bool channels_last = x.ndim() == 4 && !x.IsContiguous() && x.strides()[1] == x.GetItemSize();
    return channels_last ? chainerx::EmptyChannelsLast(shape, dtype) : chainerx::Empty(shape, dtype);
}

}  // namespace

// A dense copy in logical (row-major) order; the array itself when it already is dense.
chainerx::Array AsContiguous(const chainerx::Array& a) {
    if (a.IsContiguous()) return a;
    chainerx::Array dense = chainerx::Empty(a.shape(), a.dtype());
    chx_hip_tensor xt = a.hip(), yt = dense.hip();
    CHXVM_HIP_CALL(chx_hip_cast(&xt, &yt, chainerx::CurrentStream()));  // same element type on both sides: a strided copy
    return dense;
}

chainerx::Array GemmOp::RunImpl(
        ChxVMState* st, const chainerx::Array& a, const chainerx::Array& b, const absl::optional<chainerx::Array>& c) {
    CheckFloat32(a, "Gemm", "a");
    CheckFloat32(b, "Gemm", "b");
    CHECK_EQ(2, a.ndim()) << "Gemm: a must be a matrix";
    CHECK_EQ(2, b.ndim()) << "Gemm: b must be a matrix";
    if (c.has_value()) CheckFloat32(*c, "Gemm", "c");
    const int64_t m = a.shape()[trans_a ? 1 : 0], n = b.shape()[trans_b ? 0 : 1];
    chainerx::Array y = chainerx::Empty(chainerx::Shape{m, n}, chainerx::Dtype::kFloat32);
    chx_hip_tensor at = a.hip(), bt = b.hip(), yt = y.hip(), ct;
    if (c.has_value()) ct = c->hip();
    CHXVM_HIP_CALL(chx_hip_gemm_f32(&at, &bt, c.has_value() ? &ct : nullptr, static_cast<float>(alpha), static_cast<float>(beta),
                                    trans_a ? 1 : 0, trans_b ? 1 : 0, &yt, chainerx::CurrentStream()));
    return y;
}

// ConvOp::RunImpl, runtime/ops/connection.cc:24-30: a convolution the quantizer left in float (one with a bias).
chainerx::Array ConvOp::RunImpl(
        ChxVMState* st, const chainerx::Array& x, const chainerx::Array& w, const absl::optional<chainerx::Array>& b) {
    CheckFloat32(x, "Conv", "x");
    CheckFloat32(w, "Conv", "w");
    if (b.has_value()) CheckFloat32(*b, "Conv", "b");
    const chx_hip_conv_params p = MakeConvParams(x, w, strides, pads, group, auto_pad);
    chainerx::Array y = EmptyLike4d(x, ConvOutputShape(x, w, p), chainerx::Dtype::kFloat32);
    chx_hip_tensor xt = x.hip(), wt = w.hip(), yt = y.hip(), bt;
    if (b.has_value()) bt = b->hip();
    CHXVM_HIP_CALL(chx_hip_conv_f32(&xt, &wt, b.has_value() ? &bt : nullptr, &p, &yt, chainerx::CurrentStream()));
    return y;
}

chainerx::Array LinearOp::RunImpl(
        ChxVMState* st, const chainerx::Array& x, const chainerx::Array& w, const absl::optional<chainerx::Array>& b) {
    CheckFloat32(x, "Linear", "x");
    CheckFloat32(w, "Linear", "w");
    if (b.has_value()) CheckFloat32(*b, "Linear", "b");
    CHECK_EQ(2, w.ndim()) << "Linear: w must be [out, in]";
    CHECK(n_batch_axes >= 1 && n_batch_axes < x.ndim()) << "Linear: n_batch_axes " << n_batch_axes << " for an x of rank " << x.ndim();
    const chainerx::Array xd = AsContiguous(x);
    chainerx::Shape shape;
    for (int i = 0; i < n_batch_axes; ++i) shape.push_back(x.shape()[i]);
    shape.push_back(w.shape()[0]);
    chainerx::Array y = chainerx::Empty(shape, chainerx::Dtype::kFloat32);
    chx_hip_tensor xt = xd.hip(), wt = w.hip(), yt = y.hip(), bt;
    if (b.has_value()) bt = b->hip();
    CHXVM_HIP_CALL(chx_hip_linear_f32(&xt, &wt, b.has_value() ? &bt : nullptr, static_cast<int32_t>(n_batch_axes), &yt,
                                      chainerx::CurrentStream()));
    return y;
}

chainerx::Array FlattenOp::RunImpl(ChxVMState* st, const chainerx::Array& input) {
    const int ax = axis < 0 ? static_cast<int>(axis) + input.ndim() : static_cast<int>(axis);  // ResolveAxis, chainerx_util.cc:417-422
    CHECK_GE(ax, 0);
    CHECK_LT(ax, input.ndim());
    int64_t d0 = 1, d1 = 1;
    for (int i = 0; i < input.ndim(); ++i) (i < ax ? d0 : d1) *= input.shape()[i];
    return AsContiguous(input).Reshape(chainerx::Shape{d0, d1});
}

// ConcatOp::RunImpl, runtime/ops/manipulation.cc:74-76 (chainerx::Concatenate): every input is copied into its span of
// the result (a strided device copy each); the result is laid out like the first input when all of them are
// channels-last feature maps, dense otherwise.
chainerx::Array ConcatOp::RunImpl(ChxVMState* st, const std::vector<chainerx::Array>& inputs) {
    CHECK(!inputs.empty()) << "Concat: no inputs";
    const chainerx::Array& first = inputs[0];
    const int ax = static_cast<int>(axis < 0 ? axis + first.ndim() : axis);
    CHECK(ax >= 0 && ax < first.ndim()) << "Concat: axis " << axis << " out of range";
    chainerx::Shape shape = first.shape();
    int64_t total = 0;
    bool channels_last = true;
    for (const chainerx::Array& a : inputs) {
        CHECK(a.dtype() == first.dtype()) << "Concat: inputs of different types";
        CHECK_EQ(first.ndim(), a.ndim()) << "Concat: inputs of different rank";
        for (int d = 0; d < a.ndim(); ++d)
            if (d != ax) CHECK_EQ(first.shape()[d], a.shape()[d]) << "Concat: extents differ on axis " << d;
        total += a.shape()[ax];
        channels_last = channels_last && a.ndim() == 4 && !a.IsContiguous() && a.strides()[1] == a.GetItemSize();
    }
    shape[ax] = total;
    chainerx::Array y = channels_last ? chainerx::EmptyChannelsLast(shape, first.dtype()) : chainerx::Empty(shape, first.dtype());
    int64_t at = 0;
    for (const chainerx::Array& a : inputs) {
        if (a.shape()[ax] == 0) continue;
        const chainerx::Array span = y.Narrow(ax, at, a.shape()[ax]);
        chx_hip_tensor xt = a.hip(), yt = span.hip();
        CHXVM_HIP_CALL(chx_hip_cast(&xt, &yt, chainerx::CurrentStream()));  // same element type on both sides: a strided copy
        at += a.shape()[ax];
    }
    return y;
}

// TransposeOp::RunImpl, runtime/ops/manipulation.cc:101-107: a view; no perm reverses the axes, a perm shorter than
// the rank leaves the remaining axes in place.
chainerx::Array TransposeOp::RunImpl(ChxVMState* st, const chainerx::Array& data) {
    std::vector<int> axes;
    if (perm.empty()) {
        for (int i = data.ndim() - 1; i >= 0; --i) axes.push_back(i);
    } else {
        for (int64_t p : perm) axes.push_back(static_cast<int>(p < 0 ? p + data.ndim() : p));
        while (data.ndim() > static_cast<int>(axes.size())) axes.push_back(static_cast<int>(axes.size()));
    }
    CHECK_EQ(static_cast<size_t>(data.ndim()), axes.size()) << "Transpose: perm longer than the rank";
    std::vector<bool> seen(axes.size(), false);
    for (int a : axes) {
        CHECK(a >= 0 && a < data.ndim() && !seen[a]) << "Transpose: perm is not a permutation of the axes";
        seen[a] = true;
    }
    return data.Transpose(axes);
}

// SqueezeOp::RunImpl, runtime/ops/manipulation.cc:60-62 (chainerx::Squeeze): the named axes, which must have extent 1,
// or every axis of extent 1 when none is named.
chainerx::Array SqueezeOp::RunImpl(ChxVMState* st, const chainerx::Array& data) {
    std::vector<bool> drop(data.ndim(), false);
    if (axes.empty()) {
        for (int i = 0; i < data.ndim(); ++i) drop[i] = data.shape()[i] == 1;
    } else {
        for (int64_t a : axes) {
            const int ax = static_cast<int>(a < 0 ? a + data.ndim() : a);
            CHECK(ax >= 0 && ax < data.ndim()) << "Squeeze: axis " << a << " out of range";
            CHECK_EQ(1, data.shape()[ax]) << "Squeeze: axis " << a << " has extent " << data.shape()[ax];
            drop[ax] = true;
        }
    }
    chainerx::Shape shape;
    for (int i = 0; i < data.ndim(); ++i)
        if (!drop[i]) shape.push_back(data.shape()[i]);
    return AsContiguous(data).Reshape(shape);
}

// UnsqueezeOp::RunImpl, runtime/ops/manipulation.cc:64-72.
chainerx::Array UnsqueezeOp::RunImpl(ChxVMState* st, const chainerx::Array& data) {
    std::vector<int64_t> dims(data.shape().begin(), data.shape().end());
    for (int64_t a : axes) {
        const int64_t d = a < 0 ? static_cast<int64_t>(dims.size() + axes.size()) + a : a;
        CHECK(d >= 0 && d <= static_cast<int64_t>(dims.size())) << "Unsqueezing axis out of bound: " << d;
        dims.insert(dims.begin() + d, 1);
    }
    return AsContiguous(data).Reshape(chainerx::Shape(dims.begin(), dims.end()));
}

}  // namespace runtime
}  // namespace chainer_compiler
