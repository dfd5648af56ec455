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


_DTYPE_NAMES = {torch.float32: "float32", torch.uint8: "uint8", torch.int8: "int8"}


def fusion_program(inputs, statements, outputs):
    """Text of a fusion program (the `code` field of an ElementWiseNvrtc instruction
    emitted for the hip backend).

    inputs / outputs: list of (name, torch dtype); statements: list of
    (out_name, op, operand, ...) in topological order."""
    lines = ["chxhip-fusion 1", "in " + " ".join("%s:%s" % (n, _DTYPE_NAMES[d]) for n, d in inputs)]
    for st in statements:
        lines.append("%s = %s %s" % (st[0], st[1], " ".join(str(a) for a in st[2:])))
    lines.append("out " + " ".join("%s:%s" % (n, _DTYPE_NAMES[d]) for n, d in outputs))
    return "\n".join(lines) + "\n"


def _program_output_dtypes(code):
    names = {v: k for k, v in _DTYPE_NAMES.items()}
    for line in code.splitlines():
        t = line.split()
        if t and t[0] == "out":
            return [names[p.split(":")[1]] for p in t[1:]]
    raise ValueError("fusion program has no 'out' line")


def ElementWiseNvrtc(inputs, num_outputs, code, fusion_id=0, outs=None):
    """ElementWiseNvrtcOp::RunImpl, runtime/ops/nvrtc.cc:90-161: result shape is the
    broadcast of the input shapes; `num_outputs` arrays of that shape are allocated.
    When every full-shape input is channels-last the outputs are allocated
    channels-last too, so chains between convolutions never transpose."""
    out_dtypes = _program_output_dtypes(code)
    assert len(out_dtypes) == num_outputs
    if outs is None:
        shape = torch.broadcast_shapes(*[tuple(t.shape) for t in inputs])
        full = [t for t in inputs if tuple(t.shape) == tuple(shape)]
        cl = len(shape) == 4 and full and all(
            t.permute(0, 2, 3, 1).is_contiguous() and not t.is_contiguous() for t in full)
        if cl:
            outs = [_channels_last_empty(shape, dt, inputs[0].device) for dt in out_dtypes]
        else:
            outs = [torch.empty(shape, dtype=dt, device=inputs[0].device) for dt in out_dtypes]
    ins = capi.tensor_array([capi.desc(t) for t in inputs])
    outp = capi.tensor_array([capi.desc(t) for t in outs])
    capi.check(capi.lib().chx_hip_elementwise(code.encode(), ctypes.c_int32(fusion_id), ins,
                                              ctypes.c_int32(len(inputs)), outp, ctypes.c_int32(len(outs)),
                                              capi.stream_ptr()))
    return outs
