// Attribute helpers shared by the convolution ops (runtime/chainerx_util.cc:180-200, 276-311
// of the chainer-compiler tree).
#pragma once

#include <string>

#include "chainerx_lite.h"

namespace chainer_compiler {
namespace runtime {

typedef chainerx::StackVector<int64_t, chainerx::kMaxNdim> Int64StackVector;

// An empty strides / pads attribute means 1 / 0 for every spatial axis.
Int64StackVector ComplementStride(const Int64StackVector& strides, const chainerx::Array& input);
Int64StackVector ComplementPad(const Int64StackVector& pads, const chainerx::Array& input);

// '' (NOTSET) keeps the given begin pads (end = begin); 'SAME_UPPER' computes them so that the
// output extent is ceil(in / stride), the extra element of padding going to the end.  Returns
// begin pads, followed by end pads only when some end pad is positive -- the reference's
// convention, which GroupedConv turns into an explicit asymmetric padding.
Int64StackVector CalculateAutoPad(
        const std::string& auto_pad, const chainerx::Array& x, const Int64StackVector& kernel_shape,
        const Int64StackVector& strides, const Int64StackVector& in_pads);

// strides / begin and end pads of a 2-D convolution as the C ABI takes them.
chx_hip_conv_params MakeConvParams(
        const chainerx::Array& x, const chainerx::Array& w, const Int64StackVector& strides, const Int64StackVector& pads,
        int group, const std::string& auto_pad);

chainerx::Shape ConvOutputShape(const chainerx::Array& x, const chainerx::Array& w, const chx_hip_conv_params& p);

// The same for one or three spatial axes (the completion helpers above are rank-generic, as in the reference), with
// the result shape.
chx_hip_conv_nd_params MakeConvNdParams(
        const chainerx::Array& x, const chainerx::Array& w, const Int64StackVector& strides, const Int64StackVector& pads,
        int group, const std::string& auto_pad, chainerx::Shape* y_shape);

}  // namespace runtime
}  // namespace chainer_compiler
