"""Python mirror of the ChxVM ops on the quantized-inference path.

Each function has the name, argument order and meaning of the op's RunImpl in the
reference (runtime/ops/quantize.cc, runtime/ops/nvrtc.cc); attributes that the
generated op classes keep as members (strides, pads, group, auto_pad) are keyword
arguments.  Arrays are torch device tensors; scalars that ChxVM passes as
StrictScalar are Python numbers, with the zero point's dtype given explicitly
because it selects the output dtype (runtime/ops/quantize.cc:17-25).

All arithmetic happens in libchx_hip.so; these wrappers only infer output shapes
and allocate, like the RunImpl bodies do.
"""
import ctypes

import torch

from . import capi


def _f(v):
    return ctypes.c_float(float(v))


def _i(v):
    return ctypes.c_int32(int(v))


def _channels_last_empty(shape, dtype, device):
    n, c, h, w = shape
    return torch.empty((n, h, w, c), dtype=dtype, device=device).permute(0, 3, 1, 2)


def QuantizeLinear(x, y_scale, y_zero_point=None, zero_point_dtype=torch.uint8, flags=0, out=None):
    """QuantizeLinearOp::RunImpl, runtime/ops/quantize.cc:48-53.  An absent zero point
    means uint8 0."""
    zp = 0 if y_zero_point is None else int(y_zero_point)
    if out is None:
        out = torch.empty_like(x, dtype=zero_point_dtype)
    capi.check(capi.lib().chx_hip_quantize_linear(capi.ref(x), _f(y_scale), _i(zp), ctypes.c_uint32(flags),
                                                  capi.ref(out), capi.stream_ptr()))
    return out


def DequantizeLinear(x, x_scale, x_zero_point=None, out=None):
    """DequantizeLinearOp::RunImpl, runtime/ops/quantize.cc:55-60."""
    zp = 0 if x_zero_point is None else int(x_zero_point)
    if out is None:
        out = torch.empty_like(x, dtype=torch.float32)
    capi.check(capi.lib().chx_hip_dequantize_linear(capi.ref(x), _f(x_scale), _i(zp), capi.ref(out),
                                                    capi.stream_ptr()))
    return out
