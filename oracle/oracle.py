"""numpy face of the CPU oracle (oracle/chx_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
benchmark's cpu_baseline leg.  The product library never imports this module.

Arrays are numpy, NCHW / OIHW, C-contiguous.  Every function cites the
reference code it follows in chx_oracle.c.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libchx_oracle.so")

ROUND_REFERENCE = 0  # +0.5f then truncating cast (runtime/ops/quantize.cc:34)
ROUND_ONNX_RNE = 1   # the ONNX operator text: round-half-even, then + zero point
BIAS_NONE = 0
BIAS_REFERENCE_FLOAT = 1  # raw bias added unscaled in fp32 (runtime/ops/quantize.cc:93)
BIAS_ONNX_INT32 = 2       # int32 bias added to the accumulator

ADD, SUB, MUL, DIV = 0, 1, 2, 3


def build(force=False):
    if force or not os.path.exists(_LIB_PATH) or (
            os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_HERE, "chx_oracle.c"))):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


class _Geom(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int64) for n in (
        "N", "C", "H", "W", "OC", "KH", "KW", "sh", "sw", "ph0", "pw0", "ph1", "pw1", "group")]


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.orc_conv_out_h.restype = ctypes.c_int64
        _lib.orc_conv_out_w.restype = ctypes.c_int64
        _lib.orc_get_max_threads.restype = ctypes.c_int
    return _lib


def set_threads(n):
    lib().orc_set_threads(ctypes.c_int(int(n)))


def max_threads():
    return int(lib().orc_get_max_threads())


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _f(v):
    return ctypes.c_float(float(np.float32(v)))


def _i8flag(a):
    if a.dtype == np.int8:
        return 1
    if a.dtype == np.uint8:
        return 0
    raise TypeError("expected int8 or uint8, got %s" % a.dtype)


def _c(a, dtype=None):
    a = np.ascontiguousarray(a)
    if dtype is not None and a.dtype != dtype:
        a = a.astype(dtype)
    return a


def quantize_linear(x, y_scale, y_zero_point=0, out_dtype=np.uint8, round_mode=ROUND_REFERENCE):
    x = _c(x, np.float32)
    y = np.empty(x.shape, dtype=out_dtype)
    lib().orc_quantize_linear(_p(x), ctypes.c_int64(x.size), _f(y_scale), ctypes.c_int32(int(y_zero_point)),
                              ctypes.c_int(_i8flag(y)), ctypes.c_int(round_mode), _p(y))
    return y


def quantize_linear_multipass(x, y_scale, y_zero_point=0, out_dtype=np.uint8):
    x = _c(x, np.float32)
    y = np.empty(x.shape, dtype=out_dtype)
    tmp = np.empty(x.shape, dtype=np.float32)
    lib().orc_quantize_linear_multipass(_p(x), ctypes.c_int64(x.size), _f(y_scale), ctypes.c_int32(int(y_zero_point)),
                                        ctypes.c_int(_i8flag(y)), _p(tmp), _p(y))
    return y


def dequantize_linear(x, x_scale, x_zero_point=0, multipass=False):
    x = _c(x)
    y = np.empty(x.shape, dtype=np.float32)
    fn = lib().orc_dequantize_linear_multipass if multipass else lib().orc_dequantize_linear
    fn(_p(x), ctypes.c_int(_i8flag(x)), ctypes.c_int64(x.size), _f(x_scale), ctypes.c_int32(int(x_zero_point)), _p(y))
    return y


def _zp_arr(zp):
    if zp is None:
        return None, 0
    z = np.atleast_1d(np.asarray(zp)).astype(np.int32)
    return np.ascontiguousarray(z), z.size


def gemm(a, b, c=None, alpha=1.0, beta=1.0, trans_a=False, trans_b=False):
    """GemmOp::RunImpl, runtime/ops/math.cc:160-177."""
    a = _c(a, np.float32)
    b = _c(b, np.float32)
    M, K = (a.shape[1], a.shape[0]) if trans_a else a.shape
    K2, N = (b.shape[1], b.shape[0]) if trans_b else b.shape
    assert K == K2 and a.ndim == 2 and b.ndim == 2
    y = np.empty((M, N), dtype=np.float32)
    cp, c_rows, c_cols = None, 0, 0
    if c is not None:
        c = _c(c, np.float32)
        c2 = c.reshape((1,) * (2 - c.ndim) + c.shape)
        c_rows, c_cols = c2.shape
        assert c_rows in (1, M) and c_cols in (1, N)
        cp = _p(c)
    lib().orc_gemm_f32(_p(a), _p(b), cp, ctypes.c_int64(M), ctypes.c_int64(N), ctypes.c_int64(K), ctypes.c_int(int(trans_a)),
                       ctypes.c_int(int(trans_b)), _f(alpha), _f(beta), ctypes.c_int64(c_rows), ctypes.c_int64(c_cols), _p(y))
    return y


def linear(x, w, b=None, n_batch_axes=1):
    """LinearOp::RunImpl, runtime/ops/connection.cc:12-15 (chainerx::Linear)."""
    x = _c(x, np.float32)
    rows = int(np.prod(x.shape[:n_batch_axes]))
    y = gemm(x.reshape(rows, -1), w, b, trans_b=True)
    return y.reshape(x.shape[:n_batch_axes] + (w.shape[0],))


def flatten(x, axis=1):
    """FlattenOp::RunImpl, runtime/ops/manipulation.cc:20-28."""
    x = np.asarray(x)
    ax = axis + x.ndim if axis < 0 else axis
    assert 0 <= ax < x.ndim
    return np.ascontiguousarray(x).reshape(int(np.prod(x.shape[:ax], dtype=np.int64)), int(np.prod(x.shape[ax:], dtype=np.int64)))


def matmul_integer(a, b, a_zero_point=None, b_zero_point=None):
    a = _c(a)
    b = _c(b)
    if a.ndim <= 2:
        batch, (M, K), (K2, N) = 1, a.shape, b.shape
        out_shape = (M, N)
    else:
        assert a.shape[:-2] == b.shape[:-2]
        batch = int(np.prod(a.shape[:-2]))
        M, K = a.shape[-2:]
        K2, N = b.shape[-2:]
        out_shape = a.shape[:-2] + (M, N)
    assert K == K2
    az, azn = _zp_arr(a_zero_point)
    bz, bzn = _zp_arr(b_zero_point)
    assert azn in (0, 1, K) and bzn in (0, 1, N)
    y = np.empty(out_shape, dtype=np.int32)
    lib().orc_matmul_integer(_p(a), _i8flag(a), _p(b), _i8flag(b), ctypes.c_int64(batch), ctypes.c_int64(M),
                             ctypes.c_int64(K), ctypes.c_int64(N), _p(az) if azn else None, ctypes.c_int64(azn),
                             _p(bz) if bzn else None, ctypes.c_int64(bzn), _p(y))
    return y


def same_upper_pads(in_dim, stride, kernel):
    b, e = ctypes.c_int64(), ctypes.c_int64()
    lib().orc_same_upper_pads(ctypes.c_int64(in_dim), ctypes.c_int64(stride), ctypes.c_int64(kernel),
                              ctypes.byref(b), ctypes.byref(e))
    return b.value, e.value


def conv_geometry(x_shape, w_shape, strides=(1, 1), pads=(0, 0), group=1, auto_pad=""):
    """pads: (ph, pw) symmetric, as the emitter hands them over
    (compiler/chxvm/simple_node_emitter.cc:76-86), or (ph0, pw0, ph1, pw1)."""
    N, C, H, W = x_shape
    OC, Cg, KH, KW = w_shape
    assert C == Cg * group and OC % group == 0
    if len(pads) == 2:
        ph0, pw0, ph1, pw1 = pads[0], pads[1], pads[0], pads[1]
    else:
        ph0, pw0, ph1, pw1 = pads
    if auto_pad:
        assert auto_pad == "SAME_UPPER"
        ph0, ph1 = same_upper_pads(H, strides[0], KH)
        pw0, pw1 = same_upper_pads(W, strides[1], KW)
    g = _Geom(N, C, H, W, OC, KH, KW, strides[0], strides[1], ph0, pw0, ph1, pw1, group)
    return g


def conv_out_shape(g):
    return (g.N, g.OC, int(lib().orc_conv_out_h(ctypes.byref(g))), int(lib().orc_conv_out_w(ctypes.byref(g))))


def conv_integer(x, w, x_zero_point=None, w_zero_point=None, strides=(1, 1), pads=(0, 0), group=1, auto_pad=""):
    x = _c(x)
    w = _c(w)
    g = conv_geometry(x.shape, w.shape, strides, pads, group, auto_pad)
    wz, wzn = _zp_arr(w_zero_point)
    assert wzn in (0, 1, w.shape[0])
    y = np.empty(conv_out_shape(g), dtype=np.int32)
    lib().orc_conv_integer(_p(x), _i8flag(x), _p(w), _i8flag(w), ctypes.byref(g),
                           ctypes.c_int32(0 if x_zero_point is None else int(x_zero_point)),
                           _p(wz) if wzn else None, ctypes.c_int64(wzn), _p(y))
    return y


def _qconv(fn, x, x_scale, x_zero_point, w, w_scale, w_zero_point, y_scale, y_zero_point, y_dtype, bias, strides, pads,
           group, auto_pad, bias_mode, round_mode):
    x = _c(x)
    w = _c(w)
    g = conv_geometry(x.shape, w.shape, strides, pads, group, auto_pad)
    ws = np.ascontiguousarray(np.atleast_1d(np.asarray(w_scale, dtype=np.float32)))
    wz = np.ascontiguousarray(np.atleast_1d(np.asarray(w_zero_point)).astype(np.int32))
    assert ws.size == wz.size and ws.size in (1, w.shape[0])
    b = None if bias is None else _c(bias, np.int32)
    y = np.empty(conv_out_shape(g), dtype=y_dtype)
    fn(_p(x), _i8flag(x), _f(x_scale), ctypes.c_int32(int(x_zero_point)), _p(w), _i8flag(w), _p(ws),
       ctypes.c_int64(ws.size), _p(wz), ctypes.byref(g), _f(y_scale), ctypes.c_int32(int(y_zero_point)),
       ctypes.c_int(_i8flag(y)), _p(b) if b is not None else None, ctypes.c_int(bias_mode), ctypes.c_int(round_mode),
       _p(y))
    return y


def qlinear_conv_int(x, x_scale, x_zero_point, w, w_scale, w_zero_point, y_scale, y_zero_point, y_dtype=np.uint8,
                     bias=None, strides=(1, 1), pads=(0, 0), group=1, auto_pad="", bias_mode=BIAS_ONNX_INT32,
                     round_mode=ROUND_REFERENCE):
    return _qconv(lib().orc_qlinear_conv_int, x, x_scale, x_zero_point, w, w_scale, w_zero_point, y_scale,
                  y_zero_point, y_dtype, bias, strides, pads, group, auto_pad, bias_mode, round_mode)


def qlinear_conv_literal(x, x_scale, x_zero_point, w, w_scale, w_zero_point, y_scale, y_zero_point, y_dtype=np.uint8,
                         bias=None, strides=(1, 1), pads=(0, 0), group=1, auto_pad="",
                         bias_mode=BIAS_REFERENCE_FLOAT, round_mode=ROUND_REFERENCE):
    return _qconv(lib().orc_qlinear_conv_literal, x, x_scale, x_zero_point, w, w_scale, w_zero_point, y_scale,
                  y_zero_point, y_dtype, bias, strides, pads, group, auto_pad, bias_mode, round_mode)


def _mm_dims(a, b):
    if a.ndim <= 2:
        return 1, a.shape[0], a.shape[1], b.shape[1], (a.shape[0], b.shape[1])
    assert a.shape[:-2] == b.shape[:-2]
    return (int(np.prod(a.shape[:-2])), a.shape[-2], a.shape[-1], b.shape[-1],
            a.shape[:-2] + (a.shape[-2], b.shape[-1]))


def qlinear_matmul_int(a, a_scale, a_zero_point, b, b_scale, b_zero_point, y_scale, y_zero_point, y_dtype=np.uint8,
                       bias=None, relu=False, round_mode=ROUND_REFERENCE):
    a = _c(a)
    b = _c(b)
    batch, M, K, N, out_shape = _mm_dims(a, b)
    bi = None if bias is None else _c(bias, np.int32)
    y = np.empty(out_shape, dtype=y_dtype)
    lib().orc_qlinear_matmul_int(_p(a), _i8flag(a), _f(a_scale), ctypes.c_int32(int(a_zero_point)), _p(b), _i8flag(b),
                                 _f(b_scale), ctypes.c_int32(int(b_zero_point)), ctypes.c_int64(batch),
                                 ctypes.c_int64(M), ctypes.c_int64(K), ctypes.c_int64(N), _f(y_scale),
                                 ctypes.c_int32(int(y_zero_point)), ctypes.c_int(_i8flag(y)),
                                 _p(bi) if bi is not None else None, ctypes.c_int(1 if relu else 0),
                                 ctypes.c_int(round_mode), _p(y))
    return y


def qlinear_matmul_literal(a, a_scale, a_zero_point, b, b_scale, b_zero_point, y_scale, y_zero_point,
                           y_dtype=np.uint8, round_mode=ROUND_REFERENCE):
    a = _c(a)
    b = _c(b)
    batch, M, K, N, out_shape = _mm_dims(a, b)
    y = np.empty(out_shape, dtype=y_dtype)
    lib().orc_qlinear_matmul_literal(_p(a), _i8flag(a), _f(a_scale), ctypes.c_int32(int(a_zero_point)), _p(b),
                                     _i8flag(b), _f(b_scale), ctypes.c_int32(int(b_zero_point)),
                                     ctypes.c_int64(batch), ctypes.c_int64(M), ctypes.c_int64(K), ctypes.c_int64(N),
                                     _f(y_scale), ctypes.c_int32(int(y_zero_point)), ctypes.c_int(_i8flag(y)),
                                     ctypes.c_int(round_mode), _p(y))
    return y


# --- element-wise ops of a CPU FusionGroup: one pass, one rounding per op -----------------------

def _unary(fn, x):
    x = _c(x, np.float32)
    y = np.empty_like(x)
    fn(_p(x), ctypes.c_int64(x.size), _p(y))
    return y


def tanh(x):
    return _unary(lib().orc_tanh_f32, x)


def exp(x):
    return _unary(lib().orc_exp_f32, x)


def sigmoid(x):
    return _unary(lib().orc_sigmoid_f32, x)


def sigmoid_tanh_form(x):
    return _unary(lib().orc_sigmoid_tanh_form_f32, x)


def relu(x):
    return _unary(lib().orc_relu_f32, x)


def round_half_even(x):
    return _unary(lib().orc_round_f32, x)


def clip(x, lo, hi):
    x = _c(x, np.float32)
    y = np.empty_like(x)
    lib().orc_clip_f32(_p(x), ctypes.c_int64(x.size), _f(lo), _f(hi), _p(y))
    return y


def binary(op, a, b):
    """numpy broadcasting; operands whose flat size divides the result and that
    broadcast along leading axes only are indexed modulo (no materialisation),
    anything else is materialised first, like BroadcastTo + AsContiguous."""
    a = np.asarray(a, dtype=np.float32)
    b = np.asarray(b, dtype=np.float32)
    shape = np.broadcast_shapes(a.shape, b.shape)
    n = int(np.prod(shape)) if len(shape) else 1

    def prep(v):
        trailing = shape[len(shape) - v.ndim:] if v.ndim else ()
        if v.size == 1 or tuple(v.shape) == tuple(trailing):
            return np.ascontiguousarray(v).reshape(-1)
        return np.ascontiguousarray(np.broadcast_to(v, shape)).reshape(-1)

    af, bf = prep(a), prep(b)
    y = np.empty(shape, dtype=np.float32)
    lib().orc_binary_f32(ctypes.c_int(op), _p(af), ctypes.c_int64(af.size), _p(bf), ctypes.c_int64(bf.size),
                         ctypes.c_int64(n), _p(y))
    return y


def run_chain(program, inputs):
    """Evaluate an element-wise chain op by op, each op one full pass over a
    materialised fp32 array (compiler/chxvm/emitter.cc:697-726: a FusionGroup on the
    CPU is emitted as its individual ops).

    program: list of (out_name, op_name, arg_names_or_values...) in topological order.
      ops: Identity Add Sub Mul Div Tanh Sigmoid Exp Relu Clip(lo,hi) Const(value)
    inputs: dict name -> numpy fp32 array.  Returns the dict of all values.
    """
    env = dict(inputs)
    for stmt in program:
        out, op, args = stmt[0], stmt[1], stmt[2:]
        if op == "Const":
            env[out] = np.float32(args[0])
        elif op == "Identity":
            env[out] = np.array(env[args[0]], dtype=np.float32, copy=True)
        elif op in ("Add", "Sub", "Mul", "Div"):
            env[out] = binary({"Add": ADD, "Sub": SUB, "Mul": MUL, "Div": DIV}[op], env[args[0]], env[args[1]])
        elif op == "Tanh":
            env[out] = tanh(env[args[0]])
        elif op == "Sigmoid":
            env[out] = sigmoid(env[args[0]])
        elif op == "Exp":
            env[out] = exp(env[args[0]])
        elif op == "Relu":
            env[out] = relu(env[args[0]])
        elif op == "Clip":
            env[out] = clip(env[args[0]], args[1], args[2])
        else:
            raise ValueError("op not in the fusable set: %s" % op)
    return env


# --- pooling on quantized tensors (runtime/ops/pooling.cc:47-75 between DQ and Q) -----------------

def pool_out_dim(in_dim, p0, p1, k, s, cover_all=False):
    lib().orc_pool_out_dim.restype = ctypes.c_int64
    return int(lib().orc_pool_out_dim(*[ctypes.c_int64(v) for v in (in_dim, p0, p1, k, s)], ctypes.c_int(int(cover_all))))


def max_pool_q8(x, kernel, strides, pads=(0, 0), cover_all=False):
    x = _c(x)
    N, C, H, W = x.shape
    OH = pool_out_dim(H, pads[0], pads[0], kernel[0], strides[0], cover_all)
    OW = pool_out_dim(W, pads[1], pads[1], kernel[1], strides[1], cover_all)
    y = np.empty((N, C, OH, OW), dtype=x.dtype)
    i64 = ctypes.c_int64
    lib().orc_max_pool_q8(_p(x), _i8flag(x), i64(N), i64(C), i64(H), i64(W), i64(kernel[0]), i64(kernel[1]),
                          i64(strides[0]), i64(strides[1]), i64(pads[0]), i64(pads[1]), i64(pads[0]), i64(pads[1]),
                          ctypes.c_int(int(cover_all)), _p(y))
    return y


def max_pool(x, kernel, strides, pads=(0, 0), cover_all=False):
    """MaxPoolOp::RunImpl on float32, runtime/ops/pooling.cc:47-61."""
    x = _c(x, np.float32)
    N, C, H, W = x.shape
    OH = pool_out_dim(H, pads[0], pads[0], kernel[0], strides[0], cover_all)
    OW = pool_out_dim(W, pads[1], pads[1], kernel[1], strides[1], cover_all)
    y = np.empty((N, C, OH, OW), dtype=np.float32)
    i64 = ctypes.c_int64
    lib().orc_max_pool_f32(_p(x), i64(N), i64(C), i64(H), i64(W), i64(kernel[0]), i64(kernel[1]), i64(strides[0]), i64(strides[1]),
                           i64(pads[0]), i64(pads[1]), i64(pads[0]), i64(pads[1]), ctypes.c_int(int(cover_all)), _p(y))
    return y


def average_pool(x, kernel, strides, pads=(0, 0), count_include_pad=False):
    """AveragePoolOp::RunImpl on float32, runtime/ops/pooling.cc:63-75."""
    x = _c(x, np.float32)
    N, C, H, W = x.shape
    OH = pool_out_dim(H, pads[0], pads[0], kernel[0], strides[0])
    OW = pool_out_dim(W, pads[1], pads[1], kernel[1], strides[1])
    y = np.empty((N, C, OH, OW), dtype=np.float32)
    i64 = ctypes.c_int64
    lib().orc_average_pool_f32(_p(x), i64(N), i64(C), i64(H), i64(W), i64(kernel[0]), i64(kernel[1]), i64(strides[0]), i64(strides[1]),
                               i64(pads[0]), i64(pads[1]), ctypes.c_int(int(count_include_pad)), _p(y))
    return y


def softmax(x, axis=1, is_onnx_semantics=True):
    """SoftmaxOp::RunImpl, runtime/ops/activation.cc:66-95."""
    x = _c(x, np.float32)
    if axis < 0:
        axis += x.ndim
    outer = int(np.prod(x.shape[:axis], dtype=np.int64))
    if is_onnx_semantics:
        length, inner = int(np.prod(x.shape[axis:], dtype=np.int64)), 1
    else:
        length, inner = x.shape[axis], int(np.prod(x.shape[axis + 1:], dtype=np.int64))
    y = np.empty(x.shape, dtype=np.float32)
    i64 = ctypes.c_int64
    lib().orc_softmax_f32(_p(x), i64(outer), i64(length), i64(inner), _p(y))
    return y


def conv(x, w, bias=None, strides=(1, 1), pads=(0, 0), group=1, auto_pad=""):
    """ConvOp::RunImpl on float32, runtime/ops/connection.cc:24-30."""
    x, w = _c(x, np.float32), _c(w, np.float32)
    g = conv_geometry(x.shape, w.shape, strides, pads, group, auto_pad)
    b = None if bias is None else _c(bias, np.float32)
    y = np.empty(conv_out_shape(g), dtype=np.float32)
    lib().orc_conv_f32(_p(x), _p(w), _p(b) if b is not None else None, ctypes.byref(g), _p(y))
    return y


def fixed_batch_norm(x, s, bias, mean, var, epsilon=1e-5):
    """FixedBatchNormalizationOp::RunImpl, runtime/ops/normalization.cc:210-225, x [N, C, ...] float32."""
    x = _c(x, np.float32)
    s, bias, mean, var = (_c(np.asarray(v).reshape(-1), np.float32) for v in (s, bias, mean, var))
    N, C = x.shape[0], x.shape[1]
    inner = int(np.prod(x.shape[2:], dtype=np.int64))
    assert s.size == bias.size == mean.size == var.size == C
    y = np.empty(x.shape, dtype=np.float32)
    i64 = ctypes.c_int64
    lib().orc_fixed_batch_norm_f32(_p(x), _p(s), _p(bias), _p(mean), _p(var), ctypes.c_float(epsilon), i64(N), i64(C), i64(inner), _p(y))
    return y


def average_pool_q8(x, x_scale, x_zero_point, kernel, strides, pads, y_scale, y_zero_point, y_dtype=np.uint8,
                    count_include_pad=False, round_mode=ROUND_REFERENCE):
    x = _c(x)
    N, C, H, W = x.shape
    OH = pool_out_dim(H, pads[0], pads[0], kernel[0], strides[0])
    OW = pool_out_dim(W, pads[1], pads[1], kernel[1], strides[1])
    y = np.empty((N, C, OH, OW), dtype=y_dtype)
    i64 = ctypes.c_int64
    lib().orc_average_pool_q8(_p(x), _i8flag(x), _f(x_scale), ctypes.c_int32(int(x_zero_point)), i64(N), i64(C), i64(H),
                              i64(W), i64(kernel[0]), i64(kernel[1]), i64(strides[0]), i64(strides[1]), i64(pads[0]),
                              i64(pads[1]), ctypes.c_int(int(count_include_pad)), _f(y_scale),
                              ctypes.c_int32(int(y_zero_point)), ctypes.c_int(_i8flag(y)), ctypes.c_int(round_mode), _p(y))
    return y
