#include "chainerx_util.h"

#include <cstring>

namespace chainer_compiler {
namespace runtime {

namespace {

Int64StackVector ComplementStrideOrPad(const Int64StackVector& orig, const chainerx::Array& input, int default_value) {
    if (!orig.empty()) return orig;
    CHECK_LE(2, input.ndim()) << input.shape();
    Int64StackVector filled;
    for (int i = 0; i < input.ndim() - 2; ++i) filled.push_back(default_value);
    return filled;
}

}  // namespace

Int64StackVector ComplementStride(const Int64StackVector& strides, const chainerx::Array& input) {
    return ComplementStrideOrPad(strides, input, 1);
}

Int64StackVector ComplementPad(const Int64StackVector& pads, const chainerx::Array& input) {
    return ComplementStrideOrPad(pads, input, 0);
}

Int64StackVector CalculateAutoPad(
        const std::string& auto_pad, const chainerx::Array& x, const Int64StackVector& kernel_shape,
        const Int64StackVector& strides, const Int64StackVector& in_pads) {
    CHECK_EQ(kernel_shape.size(), in_pads.size());
    CHECK_EQ(strides.size(), in_pads.size());
    CHECK_EQ(x.shape().size(), in_pads.size() + 2);
    Int64StackVector begin = in_pads, end;
    end.resize(in_pads.size());
    bool any_end = false;
    if (!auto_pad.empty()) {
        CHECK_EQ(auto_pad, "SAME_UPPER");
        for (size_t i = 0; i < begin.size(); ++i) {
            const int64_t in_dim = x.shape()[2 + i];
            const int64_t target = (in_dim + strides[i] - 1) / strides[i];
            const int64_t needed = (target - 1) * strides[i] + kernel_shape[i] - in_dim;
            begin[i] = needed / 2;
            end[i] = needed - begin[i];
            any_end = any_end || end[i] > 0;
        }
    }
    if (any_end)
        for (int64_t e : end) begin.push_back(e);
    return begin;
}

chx_hip_conv_params MakeConvParams(
        const chainerx::Array& x, const chainerx::Array& w, const Int64StackVector& strides, const Int64StackVector& pads,
        int group, const std::string& auto_pad) {
    CHECK_EQ(4, x.ndim()) << "only 2-D convolutions on the hip backend";
    CHECK_EQ(4, w.ndim());
    const Int64StackVector st = ComplementStride(strides, x);
    const Int64StackVector pd = ComplementPad(pads, x);
    const Int64StackVector full = CalculateAutoPad(auto_pad, x, Int64StackVector{w.shape()[2], w.shape()[3]}, st, pd);
    chx_hip_conv_params p;
    p.stride_h = static_cast<int32_t>(st[0]);
    p.stride_w = static_cast<int32_t>(st[1]);
    p.pad_h_begin = static_cast<int32_t>(full[0]);
    p.pad_w_begin = static_cast<int32_t>(full[1]);
    p.pad_h_end = static_cast<int32_t>(full.size() == 4 ? full[2] : full[0]);
    p.pad_w_end = static_cast<int32_t>(full.size() == 4 ? full[3] : full[1]);
    p.group = group;
    return p;
}

chainerx::Shape ConvOutputShape(const chainerx::Array& x, const chainerx::Array& w, const chx_hip_conv_params& p) {
    const int64_t oh = (x.shape()[2] + p.pad_h_begin + p.pad_h_end - w.shape()[2]) / p.stride_h + 1;
    const int64_t ow = (x.shape()[3] + p.pad_w_begin + p.pad_w_end - w.shape()[3]) / p.stride_w + 1;
    return chainerx::Shape{x.shape()[0], w.shape()[0], oh, ow};
}

chx_hip_conv_nd_params MakeConvNdParams(
        const chainerx::Array& x, const chainerx::Array& w, const Int64StackVector& strides, const Int64StackVector& pads,
        int group, const std::string& auto_pad, chainerx::Shape* y_shape) {
    const int ns = x.ndim() - 2;
    CHECK(ns >= 1 && ns <= 3) << "convolutions over 1, 2 or 3 spatial axes on the hip backend, got an input of shape " << x.shape();
    CHECK_EQ(x.ndim(), w.ndim());
    const Int64StackVector st = ComplementStride(strides, x);
    const Int64StackVector pd = ComplementPad(pads, x);
    CHECK_EQ(static_cast<size_t>(ns), st.size());
    Int64StackVector kernel, begin_in;
    for (int i = 0; i < ns; ++i) kernel.push_back(w.shape()[2 + i]);
    // an explicit begin/end list passes through; a begin list goes through the auto-pad completion
    Int64StackVector full;
    if (pd.size() == static_cast<size_t>(2 * ns)) {
        full = pd;
    } else {
        CHECK_EQ(static_cast<size_t>(ns), pd.size());
        full = CalculateAutoPad(auto_pad, x, kernel, st, pd);
    }
    chx_hip_conv_nd_params p;
    memset(&p, 0, sizeof(p));
    p.n_spatial = ns;
    p.group = group;
    *y_shape = chainerx::Shape{x.shape()[0], w.shape()[0]};
    for (int i = 0; i < 3; ++i) p.stride[i] = 1;
    for (int i = 0; i < ns; ++i) {
        p.stride[i] = static_cast<int32_t>(st[i]);
        p.pad_begin[i] = static_cast<int32_t>(full[i]);
        p.pad_end[i] = static_cast<int32_t>(full.size() == static_cast<size_t>(2 * ns) ? full[ns + i] : full[i]);
        y_shape->push_back((x.shape()[2 + i] + p.pad_begin[i] + p.pad_end[i] - w.shape()[2 + i]) / p.stride[i] + 1);
    }
    return p;
}

}  // namespace runtime
}  // namespace chainer_compiler
