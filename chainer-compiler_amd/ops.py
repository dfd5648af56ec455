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


_DTYPE_NAMES = {torch.float32: "float32", torch.float16: "float16", torch.float64: "float64", torch.uint8: "uint8", torch.int8: "int8"}


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
    """Result types of a fusion program: this library's program text or the CUDA C text the reference's compiler emits."""
    torch_of = {v: k for k, v in capi._TORCH_TO_CHX.items()}
    return [torch_of[c] for c in capi.elementwise_output_dtypes(code)]


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


# --- convolution attribute handling (runtime/chainerx_util.cc:180-200, 276-311) -----------------

def _complement(values, ndim_spatial, default):
    """ComplementStride / ComplementPad: an empty attribute means `default` per spatial axis."""
    values = list(values)
    return values if values else [default] * ndim_spatial


def _auto_pad(auto_pad, in_shape, kernel, strides, pads):
    """CalculateAutoPad: only '' (NOTSET) and 'SAME_UPPER'; the extra padding goes to the end."""
    begin, end = list(pads), list(pads)
    if auto_pad:
        if auto_pad != "SAME_UPPER":
            raise ValueError("auto_pad must be '' or 'SAME_UPPER', got %r" % auto_pad)
        for i in range(len(pads)):
            target = (in_shape[i] + strides[i] - 1) // strides[i]
            need = (target - 1) * strides[i] + kernel[i] - in_shape[i]
            begin[i] = need // 2
            end[i] = need - begin[i]
    return begin, end


def _conv_setup(x, w, strides, pads, group, auto_pad):
    """Completed attributes and the result shape; x [N,C,H,W] gives the 2-D parameter block, x with one or three spatial
    axes the rank-generic one."""
    ns = x.dim() - 2
    strides = _complement(strides, ns, 1)
    pads = _complement(pads, ns, 0)
    if len(pads) == 2 * ns:    # explicit begin/end list (what ApplyAsymmetricPad handles)
        begin, end = pads[:ns], pads[ns:]
    else:
        begin, end = _auto_pad(auto_pad, x.shape[2:], w.shape[2:], strides, pads)
    out = tuple((x.shape[2 + i] + begin[i] + end[i] - w.shape[2 + i]) // strides[i] + 1 for i in range(ns))
    if ns == 2:
        return capi.conv_params(strides, begin, end, group), (x.shape[0], w.shape[0]) + out
    return capi.conv_nd_params(strides, begin, end, group), (x.shape[0], w.shape[0]) + out


def _alloc_like_input_layout(x, shape, dtype):
    if x.dim() == 4 and not x.is_contiguous() and x.permute(0, 2, 3, 1).is_contiguous():
        return _channels_last_empty(shape, dtype, x.device)
    return torch.empty(shape, dtype=dtype, device=x.device)


def QLinearConv(x, x_scale, x_zero_point, w, w_scale, w_zero_point, y_scale, y_zero_point, b=None, strides=(),
                pads=(), group=1, auto_pad="", zero_point_dtype=torch.uint8, flags=0, out=None):
    """QLinearConvOp::RunImpl, runtime/ops/quantize.cc:62-94.  The output dtype is the
    dtype of y_zero_point."""
    params, shape = _conv_setup(x, w, strides, pads, group, auto_pad)
    if out is None:
        out = _alloc_like_input_layout(x, shape, zero_point_dtype)
    entry = capi.lib().chx_hip_qlinear_conv if x.dim() == 4 else capi.lib().chx_hip_qlinear_conv_nd
    capi.check(entry(
        capi.ref(x), _f(x_scale), _i(x_zero_point), capi.ref(w), capi.ref(w_scale), capi.ref(w_zero_point),
        _f(y_scale), _i(y_zero_point), capi.ref(b), ctypes.byref(params), ctypes.c_uint32(flags), capi.ref(out),
        capi.stream_ptr()))
    return out


def ConvInteger(x, w, x_zero_point=None, w_zero_point=None, strides=(), pads=(), group=1, auto_pad="", out=None):
    """ConvIntegerOp::RunImpl, runtime/ops/quantize.cc:116-146."""
    params, shape = _conv_setup(x, w, strides, pads, group, auto_pad)
    if out is None:
        out = _alloc_like_input_layout(x, shape, torch.int32)
    entry = capi.lib().chx_hip_conv_integer if x.dim() == 4 else capi.lib().chx_hip_conv_integer_nd
    capi.check(entry(
        capi.ref(x), capi.ref(w), _i(0 if x_zero_point is None else x_zero_point), capi.ref(w_zero_point),
        ctypes.byref(params), capi.ref(out), capi.stream_ptr()))
    return out


def MatMulInteger(a, b, a_zero_point=None, b_zero_point=None, out=None):
    """MatMulIntegerOp::RunImpl, runtime/ops/quantize.cc:96-114."""
    if out is None:
        out = torch.empty(tuple(a.shape[:-1]) + (b.shape[-1],), dtype=torch.int32, device=a.device)
    capi.check(capi.lib().chx_hip_matmul_integer(capi.ref(a), capi.ref(b), capi.ref(a_zero_point),
                                                 capi.ref(b_zero_point), capi.ref(out), capi.stream_ptr()))
    return out


def QLinearMatMul(a, a_scale, a_zero_point, b, b_scale, b_zero_point, y_scale, y_zero_point, bias=None,
                  zero_point_dtype=torch.uint8, flags=0, out=None):
    """The DequantizeLinear, DequantizeLinear, MatMul, QuantizeLinear sequence that
    ReplaceQLinearMatMul (compiler/simplifier.cc:675-694) leaves for a QLinearMatMul
    node, as one call."""
    if out is None:
        out = torch.empty(tuple(a.shape[:-1]) + (b.shape[-1],), dtype=zero_point_dtype, device=a.device)
    capi.check(capi.lib().chx_hip_qlinear_matmul(
        capi.ref(a), _f(a_scale), _i(a_zero_point), capi.ref(b), _f(b_scale), _i(b_zero_point), _f(y_scale),
        _i(y_zero_point), capi.ref(bias), ctypes.c_uint32(flags), capi.ref(out), capi.stream_ptr()))
    return out


def BitShift(x, y, direction):
    """BitShiftOp::RunImpl, runtime/ops/quantize.cc:153-163: x << y ("LEFT") or x >> y ("RIGHT") over the broadcast of
    two integer arrays of one type."""
    assert direction in ("LEFT", "RIGHT")
    shape = torch.broadcast_shapes(tuple(x.shape), tuple(y.shape))
    z = torch.empty(shape, dtype=x.dtype, device=x.device)
    capi.check(capi.lib().chx_hip_bit_shift(capi.ref(x), capi.ref(y), ctypes.c_int32(1 if direction == "LEFT" else 0),
                                            capi.ref(z), capi.stream_ptr()))
    return z


def codes_minus_128(x, out=None):
    """chx_hip_codes_minus_128: a uint8 tensor as int8 codes minus 128 (the storage CHX_HIP_STORE_MINUS_128 writes), or
    such an int8 tensor back as uint8.  No counterpart in the reference."""
    if out is None:
        out = torch.empty_like(x, dtype=torch.int8 if x.dtype == torch.uint8 else torch.uint8)
    capi.check(capi.lib().chx_hip_codes_minus_128(capi.ref(x), capi.ref(out), capi.stream_ptr()))
    return out


def Gemm(a, b, c=None, alpha=1.0, beta=1.0, trans_a=0, trans_b=0, out=None):
    """GemmOp::RunImpl, runtime/ops/math.cc:160-177, on float32 matrices."""
    if out is None:
        m = a.shape[1] if trans_a else a.shape[0]
        n = b.shape[0] if trans_b else b.shape[1]
        out = torch.empty((m, n), dtype=torch.float32, device=a.device)
    capi.check(capi.lib().chx_hip_gemm_f32(capi.ref(a), capi.ref(b), capi.ref(c), _f(alpha), _f(beta), ctypes.c_int32(int(trans_a)),
                                           ctypes.c_int32(int(trans_b)), capi.ref(out), capi.stream_ptr()))
    return out


def Linear(x, w, b=None, n_batch_axes=1, out=None):
    """LinearOp::RunImpl, runtime/ops/connection.cc:12-15 (chainerx::Linear): x . w^T + b over the
    first n_batch_axes axes of x."""
    if out is None:
        out = torch.empty(tuple(x.shape[:n_batch_axes]) + (w.shape[0],), dtype=torch.float32, device=x.device)
    capi.check(capi.lib().chx_hip_linear_f32(capi.ref(x), capi.ref(w), capi.ref(b), ctypes.c_int32(int(n_batch_axes)), capi.ref(out),
                                             capi.stream_ptr()))
    return out


def Flatten(x, axis=1):
    """FlattenOp::RunImpl, runtime/ops/manipulation.cc:20-28: [d0 * ... * d(axis-1), the rest], the
    elements in their logical (row-major) order: a view when x is contiguous, else a device copy."""
    ax = axis + x.dim() if axis < 0 else axis
    if not 0 <= ax < x.dim():
        raise ValueError("Flatten: axis %d is outside [0, %d)" % (axis, x.dim()))
    d0 = 1
    for d in x.shape[:ax]:
        d0 *= int(d)
    if not x.is_contiguous():
        dense = torch.empty(tuple(x.shape), dtype=x.dtype, device=x.device)
        capi.check(capi.lib().chx_hip_cast(capi.ref(x), capi.ref(dense), capi.stream_ptr()))  # same type: a strided copy
        x = dense
    return x.view(d0, -1)


class QLinearConvPlan(object):
    """Weight-side state of one QLinearConv instruction (chx_hip_qconv_plan): repacked
    weights and per-channel sums, built once and reused by every run."""

    def __init__(self, w, w_scale, w_zero_point, b=None, strides=(), pads=(), group=1, auto_pad=""):
        self._keep = (w, w_scale, w_zero_point, b)
        self.w, self.strides, self.pads, self.group, self.auto_pad = w, strides, pads, group, auto_pad
        self._plans = {}

    def _plan_for(self, x):
        params, shape = _conv_setup(x, self.w, self.strides, self.pads, self.group, self.auto_pad)
        key = tuple(getattr(params, f) for f, _ in params._fields_)
        if key not in self._plans:
            handle = ctypes.c_void_p()
            w, w_scale, w_zero_point, b = self._keep
            capi.check(capi.lib().chx_hip_qconv_plan_create(
                capi.ref(w), capi.ref(w_scale), capi.ref(w_zero_point), capi.ref(b), ctypes.byref(params),
                capi.stream_ptr(), ctypes.byref(handle)))
            self._plans[key] = handle
        return self._plans[key], shape

    def run(self, x, x_scale, x_zero_point, y_scale, y_zero_point, zero_point_dtype=torch.uint8, flags=0, out=None):
        handle, shape = self._plan_for(x)
        if out is None:
            out = _alloc_like_input_layout(x, shape, zero_point_dtype)
        capi.check(capi.lib().chx_hip_qconv_plan_run(
            handle, capi.ref(x), _f(x_scale), _i(x_zero_point), _f(y_scale), _i(y_zero_point),
            ctypes.c_uint32(flags), capi.ref(out), capi.stream_ptr()))
        return out

    def run_add(self, x, x_scale, x_zero_point, y_scale, y_zero_point, r, r_scale, r_zero_point, out_scale,
                out_zero_point, relu, zero_point_dtype=torch.uint8, flags=0, out=None):
        """QLinearConv followed by QuantizeLinear(act(DequantizeLinear(y) + DequantizeLinear(r))) as
        one kernel (chx_hip_qconv_plan_run_add); `zero_point_dtype` is the type of the convolution's
        own result y, which is not written.  Raises ChxHipError with code EUNSUPPORTED when the
        weights or layouts do not fit; run the two ops separately then."""
        handle, shape = self._plan_for(x)
        if out is None:
            out = _alloc_like_input_layout(r, shape, r.dtype)
        capi.check(capi.lib().chx_hip_qconv_plan_run_add(
            handle, capi.ref(x), _f(x_scale), _i(x_zero_point), _f(y_scale), _i(y_zero_point),
            _i(capi._TORCH_TO_CHX[zero_point_dtype]), ctypes.c_uint32(flags), capi.ref(r), _f(r_scale), _i(r_zero_point),
            _f(out_scale), _i(out_zero_point), _i(1 if relu else 0), capi.ref(out), capi.stream_ptr()))
        return out

    def run_pair(self, x, x_scale, x_zero_point, split, y1_scale, y1_zero_point, y2_scale, y2_zero_point,
                 zero_point_dtypes=(torch.uint8, torch.uint8), flags=(0, 0), outs=None):
        """Two QLinearConv of the same x in one launch (chx_hip_qconv_plan_run_pair): this plan holds both filter sets
        concatenated along the output channels; the first `split` channels go to the first result with the first
        quantization, the others to the second.  Raises ChxHipError with code EUNSUPPORTED when the weights or layouts
        do not fit; run two plans then."""
        handle, shape = self._plan_for(x)
        if outs is None:
            outs = (_alloc_like_input_layout(x, (shape[0], split) + tuple(shape[2:]), zero_point_dtypes[0]),
                    _alloc_like_input_layout(x, (shape[0], shape[1] - split) + tuple(shape[2:]), zero_point_dtypes[1]))
        capi.check(capi.lib().chx_hip_qconv_plan_run_pair(
            handle, capi.ref(x), _f(x_scale), _i(x_zero_point), _i(split), _f(y1_scale), _i(y1_zero_point),
            ctypes.c_uint32(flags[0]), capi.ref(outs[0]), _f(y2_scale), _i(y2_zero_point), ctypes.c_uint32(flags[1]),
            capi.ref(outs[1]), capi.stream_ptr()))
        return outs

    def describe(self):
        """The launch configurations measured so far (chx_hip_qconv_plan_describe), one per line."""
        lines = []
        for handle in self._plans.values():
            buf = ctypes.create_string_buffer(4096)
            capi.check(capi.lib().chx_hip_qconv_plan_describe(handle, buf, ctypes.c_size_t(len(buf))))
            lines += [l for l in buf.value.decode().splitlines() if l]
        return lines

    def close(self):
        for handle in self._plans.values():
            capi.lib().chx_hip_qconv_plan_destroy(handle)
        self._plans = {}

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def _pool_out(in_dim, p0, p1, k, s, cover_all):
    if cover_all:
        return (in_dim + p0 + p1 - k + s - 1) // s + 1
    return (in_dim + p0 + p1 - k) // s + 1


def MaxPool(x, kernel_shape, strides=(), pads=(), cover_all=False, out=None):
    """MaxPoolOp::RunImpl on a float32 array, runtime/ops/pooling.cc:47-61 (the result; the op's second output,
    the context for a backward pass, has no use in inference)."""
    strides = _complement(strides, 2, 1)
    pads = _complement(pads, 2, 0)
    if out is None:
        shape = (x.shape[0], x.shape[1], _pool_out(x.shape[2], pads[0], pads[0], kernel_shape[0], strides[0], cover_all),
                 _pool_out(x.shape[3], pads[1], pads[1], kernel_shape[1], strides[1], cover_all))
        out = _alloc_like_input_layout(x, shape, torch.float32)
    capi.check(capi.lib().chx_hip_max_pool_f32(
        capi.ref(x), _i(kernel_shape[0]), _i(kernel_shape[1]), _i(strides[0]), _i(strides[1]), _i(pads[0]), _i(pads[1]),
        _i(pads[0]), _i(pads[1]), _i(1 if cover_all else 0), capi.ref(out), capi.stream_ptr()))
    return out


def AveragePool(x, kernel_shape, strides=(), pads=(), count_include_pad=False, out=None):
    """AveragePoolOp::RunImpl on a float32 array, runtime/ops/pooling.cc:63-75."""
    strides = _complement(strides, 2, 1)
    pads = _complement(pads, 2, 0)
    if out is None:
        shape = (x.shape[0], x.shape[1], _pool_out(x.shape[2], pads[0], pads[0], kernel_shape[0], strides[0], False),
                 _pool_out(x.shape[3], pads[1], pads[1], kernel_shape[1], strides[1], False))
        out = _alloc_like_input_layout(x, shape, torch.float32)
    capi.check(capi.lib().chx_hip_average_pool_f32(
        capi.ref(x), _i(kernel_shape[0]), _i(kernel_shape[1]), _i(strides[0]), _i(strides[1]), _i(pads[0]), _i(pads[1]),
        _i(1 if count_include_pad else 0), capi.ref(out), capi.stream_ptr()))
    return out


def Conv(x, w, b=None, strides=(), pads=(), group=1, auto_pad="", out=None):
    """ConvOp::RunImpl on float32, runtime/ops/connection.cc:24-30."""
    params, shape = _conv_setup(x, w, strides, pads, group, auto_pad)
    if out is None:
        out = _alloc_like_input_layout(x, shape, torch.float32)
    capi.check(capi.lib().chx_hip_conv_f32(capi.ref(x), capi.ref(w), capi.ref(b), ctypes.byref(params), capi.ref(out), capi.stream_ptr()))
    return out


def Softmax(x, axis=1, is_onnx_semantics=True, out=None):
    """SoftmaxOp::RunImpl, runtime/ops/activation.cc:66-95, on a contiguous float32 array."""
    if out is None:
        out = torch.empty_like(x)
    capi.check(capi.lib().chx_hip_softmax_f32(capi.ref(x), _i(axis), _i(1 if is_onnx_semantics else 0), capi.ref(out), capi.stream_ptr()))
    return out


def FixedBatchNormalization(x, s, bias, mean, var, epsilon=1e-5, out=None):
    """FixedBatchNormalizationOp::RunImpl, runtime/ops/normalization.cc:210-225: BatchNormalization with stored
    statistics on a float32 array [N, C, ...]."""
    if out is None:
        out = torch.empty_like(x)
    capi.check(capi.lib().chx_hip_fixed_batch_norm_f32(
        capi.ref(x), capi.ref(s), capi.ref(bias), capi.ref(mean), capi.ref(var), _f(epsilon), capi.ref(out), capi.stream_ptr()))
    return out


def MaxPoolQ8(x, kernel_shape, strides=(), pads=(), cover_all=False, out=None):
    """DequantizeLinear -> MaxPool (runtime/ops/pooling.cc:47-61) -> QuantizeLinear with equal
    quantization parameters, on the 8-bit codes: their maximum m for uint8, m + (m < 0) for int8 (the
    QuantizeLinear adds 0.5 and truncates toward zero)."""
    strides = _complement(strides, 2, 1)
    pads = _complement(pads, 2, 0)
    if out is None:
        shape = (x.shape[0], x.shape[1], _pool_out(x.shape[2], pads[0], pads[0], kernel_shape[0], strides[0], cover_all),
                 _pool_out(x.shape[3], pads[1], pads[1], kernel_shape[1], strides[1], cover_all))
        out = _alloc_like_input_layout(x, shape, x.dtype)
    capi.check(capi.lib().chx_hip_max_pool_q8(
        capi.ref(x), _i(kernel_shape[0]), _i(kernel_shape[1]), _i(strides[0]), _i(strides[1]), _i(pads[0]), _i(pads[1]),
        _i(pads[0]), _i(pads[1]), _i(1 if cover_all else 0), capi.ref(out), capi.stream_ptr()))
    return out


def AveragePoolQ8(x, x_scale, x_zero_point, kernel_shape, strides, pads, y_scale, y_zero_point,
                  count_include_pad=False, zero_point_dtype=torch.uint8, flags=0, out=None):
    """DequantizeLinear -> AveragePool (runtime/ops/pooling.cc:63-75) -> QuantizeLinear."""
    strides = _complement(strides, 2, 1)
    pads = _complement(pads, 2, 0)
    if out is None:
        shape = (x.shape[0], x.shape[1], _pool_out(x.shape[2], pads[0], pads[0], kernel_shape[0], strides[0], False),
                 _pool_out(x.shape[3], pads[1], pads[1], kernel_shape[1], strides[1], False))
        out = _alloc_like_input_layout(x, shape, zero_point_dtype)
    capi.check(capi.lib().chx_hip_average_pool_q8(
        capi.ref(x), _f(x_scale), _i(x_zero_point), _i(kernel_shape[0]), _i(kernel_shape[1]), _i(strides[0]),
        _i(strides[1]), _i(pads[0]), _i(pads[1]), _i(1 if count_include_pad else 0), _f(y_scale), _i(y_zero_point),
        ctypes.c_uint32(flags), capi.ref(out), capi.stream_ptr()))
    return out
