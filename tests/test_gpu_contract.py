"""QLinearConv, ConvInteger, MatMulInteger and QLinearMatMul on the MI355X through the
C ABI, bit-exact against the integer-accumulating CPU oracle; the literal fp32 oracle
is compared where both are provably identical and reported otherwise."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

TDT = {np.uint8: torch.uint8, np.int8: torch.int8}


@pytest.fixture(scope="module")
def g():
    import gpu_util
    gpu_util.capi.init(0)
    return gpu_util


def rand_q(rng, shape, dtype):
    lo, hi = (0, 256) if dtype == np.uint8 else (-128, 128)
    return rng.integers(lo, hi, size=shape).astype(dtype)


# ---- known-answer vectors of the ONNX node tests --------------------------------------------

def test_onnx_qlinearconv(g, onnx_vectors):
    t = onnx_vectors["test_qlinearconv"]
    x = g.dev(np.array(t["x"], np.uint8).reshape(t["x_shape"]))
    w = g.dev(np.array(t["w"], np.uint8).reshape(t["w_shape"]))
    y = g.ops.QLinearConv(x, t["x_scale"], t["x_zero_point"], w, g.dev(np.array(t["w_scale"], np.float32)),
                          g.dev(np.array(t["w_zero_point"], np.uint8)), t["y_scale"], t["y_zero_point"])
    assert g.host(y).reshape(7, 7).tolist() == t["y"]


@pytest.mark.parametrize("name", ["test_qlinearmatmul_2D", "test_qlinearmatmul_3D"])
def test_onnx_qlinearmatmul(g, onnx_vectors, name):
    t = onnx_vectors[name]
    y = g.ops.QLinearMatMul(g.dev(np.array(t["a"], np.uint8)), t["a_scale"], t["a_zero_point"],
                            g.dev(np.array(t["b"], np.uint8)), t["b_scale"], t["b_zero_point"], t["y_scale"],
                            t["y_zero_point"])
    assert g.host(y).tolist() == t["y"]


def test_onnx_matmulinteger(g, onnx_vectors):
    t = onnx_vectors["test_matmulinteger"]
    y = g.ops.MatMulInteger(g.dev(np.array(t["a"], np.uint8)), g.dev(np.array(t["b"], np.uint8)),
                            g.dev(np.array([t["a_zero_point"]], np.uint8)), g.dev(np.array([t["b_zero_point"]], np.uint8)))
    assert y.dtype == torch.int32 and g.host(y).tolist() == t["y"]


@pytest.mark.parametrize("name", ["test_basic_convinteger", "test_convinteger_with_padding"])
def test_onnx_convinteger(g, onnx_vectors, name):
    t = onnx_vectors[name]
    x = g.dev(np.array(t["x"], np.uint8).reshape(t["x_shape"]))
    w = g.dev(np.array(t["w"], np.uint8).reshape(t["w_shape"]))
    y = g.ops.ConvInteger(x, w, t["x_zero_point"], None, pads=t["pads"])
    assert list(y.shape) == t["y_shape"] and g.host(y).reshape(-1).tolist() == t["y"]


# ---- random cases against the oracle ---------------------------------------------------------

CONV_CASES = [
    # N, C, H, W, OC, KH, KW, strides, pads, group, auto_pad
    (2, 4, 7, 6, 6, 3, 3, (1, 1), (1, 1), 1, ""),
    (1, 6, 9, 8, 4, 3, 2, (2, 1), (0, 1), 2, ""),
    (2, 8, 5, 5, 8, 3, 3, (1, 1), (1, 1), 8, ""),        # depthwise
    (1, 3, 23, 23, 5, 7, 7, (2, 2), (3, 3), 1, ""),      # stem-like
    (1, 5, 6, 7, 3, 1, 1, (2, 2), (0, 0), 1, ""),        # strided pointwise
    (1, 2, 5, 4, 2, 3, 3, (2, 2), (0, 0), 1, "SAME_UPPER"),  # asymmetric end padding
    (2, 16, 6, 6, 32, 3, 3, (1, 1), (), 1, ""),          # empty pads attribute -> 0
    (1, 64, 8, 8, 64, 3, 3, (), (1, 1), 1, ""),          # empty strides attribute -> 1
]


@pytest.mark.parametrize("case", CONV_CASES)
@pytest.mark.parametrize("xdt,wdt", [(np.uint8, np.int8), (np.uint8, np.uint8), (np.int8, np.int8)])
def test_conv_integer(g, oracle, case, xdt, wdt):
    N, C, H, W, OC, KH, KW, strides, pads, group, auto_pad = case
    rng = np.random.default_rng(21)
    x, w = rand_q(rng, (N, C, H, W), xdt), rand_q(rng, (OC, C // group, KH, KW), wdt)
    wz = rand_q(rng, (OC,), wdt)
    xz = int(rand_q(rng, (1,), xdt)[0])
    kw = dict(strides=strides or (1, 1), pads=pads or (0, 0), group=group, auto_pad=auto_pad)
    want = oracle.conv_integer(x, w, xz, wz, **kw)
    got = g.ops.ConvInteger(g.dev(x), g.dev(w), xz, g.dev(wz), strides=strides, pads=pads, group=group, auto_pad=auto_pad)
    np.testing.assert_array_equal(g.host(got), want)
    # scalar weight zero point, channels-last input view
    want = oracle.conv_integer(x, w, xz, wz[:1], **kw)
    got = g.ops.ConvInteger(g.to_channels_last(g.dev(x)), g.dev(w), xz, g.dev(wz[:1].reshape(())), strides=strides,
                            pads=pads, group=group, auto_pad=auto_pad)
    np.testing.assert_array_equal(g.host(got), want)
    # no zero points at all
    np.testing.assert_array_equal(
        g.host(g.ops.ConvInteger(g.dev(x), g.dev(w), strides=strides, pads=pads, group=group, auto_pad=auto_pad)),
        oracle.conv_integer(x, w, None, None, **kw))


@pytest.mark.parametrize("case", CONV_CASES)
@pytest.mark.parametrize("bias_mode", ["none", "reference_float", "onnx_int32"])
@pytest.mark.parametrize("ydt", [np.uint8, np.int8])
def test_qlinear_conv(g, oracle, case, bias_mode, ydt):
    N, C, H, W, OC, KH, KW, strides, pads, group, auto_pad = case
    rng = np.random.default_rng(22)
    x = rand_q(rng, (N, C, H, W), np.uint8)
    w = rng.integers(-127, 128, size=(OC, C // group, KH, KW)).astype(np.int8)
    ws = rng.uniform(0.001, 0.01, size=OC).astype(np.float32)
    wz = np.zeros(OC, np.int8)
    bias = rng.integers(-1000, 1001, size=OC).astype(np.int32)
    K = (C // group) * KH * KW
    ys = np.float32(0.02 * 0.005 * 128 * 64 * np.sqrt(K) / 100)
    yz = 128 if ydt == np.uint8 else -3
    okw = dict(strides=strides or (1, 1), pads=pads or (0, 0), group=group, auto_pad=auto_pad)
    flags, b = 0, None
    if bias_mode == "reference_float":
        b, okw["bias"], okw["bias_mode"] = bias, bias, oracle.BIAS_REFERENCE_FLOAT
    elif bias_mode == "onnx_int32":
        b, okw["bias"], okw["bias_mode"] = bias, bias, oracle.BIAS_ONNX_INT32
        flags = g.capi.BIAS_ONNX_INT32
    want = oracle.qlinear_conv_int(x, 0.02, 128, w, ws, wz, ys, yz, ydt, **okw)
    got = g.ops.QLinearConv(g.dev(x), 0.02, 128, g.dev(w), g.dev(ws), g.dev(wz), ys, yz,
                            None if b is None else g.dev(b), strides=strides, pads=pads, group=group,
                            auto_pad=auto_pad, zero_point_dtype=TDT[ydt], flags=flags)
    np.testing.assert_array_equal(g.host(got), want)
    if bias_mode != "reference_float":
        assert want.min() < want.max()
    # channels-last in -> channels-last out, fused Relu, ONNX rounding
    fl = flags | g.capi.FUSE_RELU | g.capi.ROUND_ONNX_RNE
    want2 = np.maximum(oracle.qlinear_conv_int(x, 0.02, 128, w, ws, wz, ys, yz, ydt, round_mode=oracle.ROUND_ONNX_RNE,
                                               **okw), yz).astype(ydt)
    got2 = g.ops.QLinearConv(g.to_channels_last(g.dev(x)), 0.02, 128, g.dev(w), g.dev(ws), g.dev(wz), ys, yz,
                             None if b is None else g.dev(b), strides=strides, pads=pads, group=group,
                             auto_pad=auto_pad, zero_point_dtype=TDT[ydt], flags=fl)
    assert got2.permute(0, 2, 3, 1).is_contiguous()
    np.testing.assert_array_equal(g.host(got2), want2)


def test_qlinear_conv_per_tensor_and_weight_zero_points(g, oracle):
    rng = np.random.default_rng(23)
    x = rand_q(rng, (2, 8, 9, 9), np.int8)
    w = rand_q(rng, (12, 8, 3, 3), np.uint8)
    for ws, wz in ((np.float32(0.004), np.uint8(131)),
                   (rng.uniform(0.001, 0.01, size=12).astype(np.float32), rand_q(rng, (12,), np.uint8))):
        want = oracle.qlinear_conv_int(x, 0.03, -5, w, ws, wz, 0.9, 100, np.uint8, pads=(1, 1))
        got = g.ops.QLinearConv(g.dev(x), 0.03, -5, g.dev(w), g.dev(np.asarray(ws)), g.dev(np.asarray(wz)), 0.9, 100,
                                pads=(1, 1))
        np.testing.assert_array_equal(g.host(got), want)
        assert want.min() < want.max()


def test_qlinear_conv_equals_literal_reference_on_power_of_two_scales(g, oracle):
    """Where the reference's fp32 contraction is exact (power-of-two scales, |acc| < 2^24) the
    device result must equal the literal restatement of QLinearConvOp bit for bit, including
    the reference's unscaled float bias."""
    rng = np.random.default_rng(24)
    x = rand_q(rng, (2, 16, 10, 10), np.uint8)
    w = rng.integers(-127, 128, size=(24, 16, 3, 3)).astype(np.int8)
    ws = (2.0 ** rng.integers(-9, -5, size=24)).astype(np.float32)
    wz = np.zeros(24, np.int8)
    bias = rng.integers(-20, 21, size=24).astype(np.int32)
    want = oracle.qlinear_conv_literal(x, 2.0 ** -6, 128, w, ws, wz, 2.0 ** -2, 128, np.uint8, bias=bias, pads=(1, 1))
    got = g.ops.QLinearConv(g.dev(x), 2.0 ** -6, 128, g.dev(w), g.dev(ws), g.dev(wz), 2.0 ** -2, 128, g.dev(bias),
                            pads=(1, 1))
    np.testing.assert_array_equal(g.host(got), want)
    assert want.min() < want.max()


@pytest.mark.parametrize("adt,bdt", [(np.uint8, np.int8), (np.uint8, np.uint8), (np.int8, np.int8)])
@pytest.mark.parametrize("shape", [((5, 37), (37, 11)), ((3, 5, 37), (3, 37, 11)), ((32, 784), (784, 100)),
                                   ((2, 2, 4, 16), (2, 2, 16, 8))])
def test_matmul_integer(g, oracle, adt, bdt, shape):
    rng = np.random.default_rng(25)
    a, b = rand_q(rng, shape[0], adt), rand_q(rng, shape[1], bdt)
    az, bz = rand_q(rng, (1,), adt), rand_q(rng, (shape[1][-1],), bdt)
    want = oracle.matmul_integer(a, b, az, bz)
    got = g.ops.MatMulInteger(g.dev(a), g.dev(b), g.dev(az), g.dev(bz))
    np.testing.assert_array_equal(g.host(got), want)
    ak = rand_q(rng, (shape[0][-1],), adt)   # 1-D a zero point lines up with K (plain broadcasting)
    np.testing.assert_array_equal(g.host(g.ops.MatMulInteger(g.dev(a), g.dev(b), g.dev(ak), None)),
                                  oracle.matmul_integer(a, b, ak, None))
    # transposed (strided) operand
    bt = g.dev(np.ascontiguousarray(np.swapaxes(b, -1, -2))).transpose(-1, -2)
    np.testing.assert_array_equal(g.host(g.ops.MatMulInteger(g.dev(a), bt, None, g.dev(bz))),
                                  oracle.matmul_integer(a, b, None, bz))


def test_mlp_configuration(g, oracle):
    """MLP 784-100-100-10, batch 32: QuantizeLinear -> (QLinearMatMul + bias + Relu) x2 ->
    QLinearMatMul -> DequantizeLinear; uint8 activations zp 128 scale 1/255, int8 symmetric
    per-tensor weights from N(0, 0.05), int32 bias."""
    rng = np.random.default_rng(0)
    x = rng.uniform(0, 1, size=(32, 784)).astype(np.float32)
    dims = [784, 100, 100, 10]
    s_act = np.float32(1 / 255)
    h_d = g.ops.QuantizeLinear(g.dev(x), s_act, 128, torch.uint8)
    h_o = oracle.quantize_linear(x, s_act, 128, np.uint8)
    for i in range(3):
        wf = (rng.standard_normal((dims[i], dims[i + 1])) * 0.05).astype(np.float32)
        # compiler/quantize.cc:77-81: scale = 2 max|w| / 254, q = rint(w / scale)
        s_w = np.float32(np.float32(np.abs(wf).max() * 2) / np.float32(254))
        wq = np.rint(wf / s_w).astype(np.int8)
        bias = rng.integers(-2000, 2000, size=dims[i + 1]).astype(np.int32)
        relu = i < 2
        s_y = np.float32(s_act * 8)
        h_o = oracle.qlinear_matmul_int(h_o, s_act if i == 0 else s_prev, 128, wq, s_w, 0, s_y, 128, bias=bias, relu=relu)
        h_d = g.ops.QLinearMatMul(h_d, s_act if i == 0 else s_prev, 128, g.dev(wq), s_w, 0, s_y, 128, g.dev(bias),
                                  flags=g.capi.FUSE_RELU if relu else 0)
        s_prev = s_y
        np.testing.assert_array_equal(g.host(h_d), h_o)
        assert h_o.min() < h_o.max()
    out = g.ops.DequantizeLinear(h_d, s_prev, 128)
    np.testing.assert_array_equal(g.host(out), oracle.dequantize_linear(h_o, s_prev, 128))


def test_errors(g):
    x = torch.zeros((1, 4, 5, 5), dtype=torch.uint8, device="cuda")
    w = torch.zeros((6, 4, 3, 3), dtype=torch.int8, device="cuda")
    ws = torch.ones(6, device="cuda")
    wz = torch.zeros(6, dtype=torch.int8, device="cuda")
    with pytest.raises(g.capi.ChxHipError, match="expected \\[1,6,3,3\\]"):
        g.ops.QLinearConv(x, 1.0, 0, w, ws, wz, 1.0, 0, out=torch.zeros((1, 6, 5, 5), dtype=torch.uint8, device="cuda"))
    with pytest.raises(g.capi.ChxHipError, match="channels"):
        g.ops.QLinearConv(x, 1.0, 0, w, ws, wz, 1.0, 0, group=2)
    with pytest.raises(g.capi.ChxHipError, match="same shape"):
        g.ops.QLinearConv(x, 1.0, 0, w, ws, wz[:1], 1.0, 0)
    with pytest.raises(g.capi.ChxHipError, match="bias must be int32"):
        g.ops.QLinearConv(x, 1.0, 0, w, ws, wz, 1.0, 0, torch.zeros(6, device="cuda"))
    with pytest.raises(g.capi.ChxHipError, match="inner dimensions"):
        g.ops.MatMulInteger(torch.zeros((2, 3), dtype=torch.uint8, device="cuda"),
                            torch.zeros((4, 5), dtype=torch.uint8, device="cuda"),
                            out=torch.zeros((2, 5), dtype=torch.int32, device="cuda"))


@pytest.mark.parametrize("xdt", [np.uint8, np.int8])
@pytest.mark.parametrize("case", [
    # N, C, H, W, stride, pad
    (2, 32, 9, 10, 1, 1), (1, 96, 13, 12, 2, 1), (2, 16, 7, 7, 1, 0), (1, 144, 5, 6, 2, 0), (1, 48, 4, 4, 1, 1),
    # 14, 28, 21 and 7 output rows (strips of 7), 56 (strips of 14), a stride the row reuse does not cover, strides that differ
    (1, 16, 14, 5, 1, 1), (1, 16, 30, 3, 1, 0), (1, 16, 21, 4, 1, 1), (1, 16, 7, 9, 1, 1), (1, 16, 58, 3, 1, 0),
    (1, 32, 11, 10, 3, 1), (1, 16, 12, 9, (2, 1), 1), (1, 16, 9, 12, (1, 3), 1)])
def test_depthwise_qlinear_conv(g, oracle, case, xdt):
    """Depthwise 3x3 on channels-last operands (the row-packing kernel), stateless call and plan,
    both bias modes, fused Relu in both roundings; NCHW operands take the generic kernel and must
    give the same bytes."""
    N, C, H, W, stride, pad = case
    stride = stride if isinstance(stride, tuple) else (stride, stride)
    rng = np.random.default_rng(31)
    x = rand_q(rng, (N, C, H, W), xdt)
    w = rng.integers(-127, 128, size=(C, 1, 3, 3)).astype(np.int8)
    ws = rng.uniform(0.002, 0.02, size=C).astype(np.float32)
    wz = np.zeros(C, np.int8)
    bias = rng.integers(-300, 301, size=C).astype(np.int32)
    xz = 117 if xdt == np.uint8 else -11
    ys = np.float32(0.02 * 0.01 * 128 * 64 * 3 / 40)
    kw = dict(strides=stride, pads=(pad, pad), group=C)
    for bias_mode, flags in ((oracle.BIAS_ONNX_INT32, g.capi.BIAS_ONNX_INT32), (oracle.BIAS_REFERENCE_FLOAT, 0)):
        want = oracle.qlinear_conv_int(x, 0.02, xz, w, ws, wz, ys, 120, np.uint8, bias=bias, bias_mode=bias_mode, **kw)
        assert want.min() < want.max()
        xd = g.to_channels_last(g.dev(x))
        got = g.ops.QLinearConv(xd, 0.02, xz, g.dev(w), g.dev(ws), g.dev(wz), ys, 120, g.dev(bias), flags=flags, **kw)
        assert got.permute(0, 2, 3, 1).is_contiguous()
        np.testing.assert_array_equal(g.host(got), want)
        got_nchw = g.ops.QLinearConv(g.dev(x), 0.02, xz, g.dev(w), g.dev(ws), g.dev(wz), ys, 120, g.dev(bias), flags=flags, **kw)
        np.testing.assert_array_equal(g.host(got_nchw), want)
        plan = g.ops.QLinearConvPlan(g.dev(w), g.dev(ws), g.dev(wz), g.dev(bias), **kw)
        for _ in range(2):
            np.testing.assert_array_equal(g.host(plan.run(xd, 0.02, xz, ys, 120, flags=flags)), want)
        plan.close()
    # int8 output, fused Relu, ONNX rounding
    fl = g.capi.BIAS_ONNX_INT32 | g.capi.FUSE_RELU | g.capi.ROUND_ONNX_RNE
    want = np.maximum(oracle.qlinear_conv_int(x, 0.02, xz, w, ws, wz, ys, -5, np.int8, bias=bias, bias_mode=oracle.BIAS_ONNX_INT32,
                                              round_mode=oracle.ROUND_ONNX_RNE, **kw), -5).astype(np.int8)
    got = g.ops.QLinearConv(g.to_channels_last(g.dev(x)), 0.02, xz, g.dev(w), g.dev(ws), g.dev(wz), ys, -5, g.dev(bias),
                            zero_point_dtype=torch.int8, flags=fl, **kw)
    np.testing.assert_array_equal(g.host(got), want)
    # uint8 output in the reference's rounding with the Relu folded into the lower bound
    want = np.maximum(oracle.qlinear_conv_int(x, 0.02, xz, w, ws, wz, ys, 120, np.uint8, bias=bias, bias_mode=oracle.BIAS_REFERENCE_FLOAT, **kw),
                      120).astype(np.uint8)
    got = g.ops.QLinearConv(g.to_channels_last(g.dev(x)), 0.02, xz, g.dev(w), g.dev(ws), g.dev(wz), ys, 120, g.dev(bias),
                            flags=g.capi.FUSE_RELU, **kw)
    np.testing.assert_array_equal(g.host(got), want)
    assert (want > 120).any() and (want == 120).any()


@pytest.mark.parametrize("xdt", [np.uint8, np.int8])
@pytest.mark.parametrize("case", [
    # N, C, H, W, OC, KH, KW, stride, pad
    (2, 3, 37, 41, 64, 7, 7, 2, 3),     # ResNet stem geometry, ragged tiles
    (1, 3, 33, 30, 32, 3, 3, 2, 1),     # MobileNetV2 stem geometry: 4-byte filter rows, half an output-channel block
    (1, 1, 20, 20, 10, 5, 5, 1, 2),     # one channel, stride 1
    (2, 4, 17, 19, 96, 3, 3, 1, 1),     # two output-channel blocks
    (1, 3, 16, 50, 130, 7, 7, 2, 3),    # three blocks, the last with 2 channels
    (1, 2, 9, 12, 7, 8, 8, 1, 0),       # filter rows of exactly 8 bytes
    (1, 8, 12, 12, 16, 4, 4, 2, 1),     # C * KH = 32, the most K groups
    (1, 3, 9, 9, 8, 3, 3, 3, 0),        # stride 3
])
def test_planar_input_qlinear_conv(g, oracle, case, xdt):
    """Few input channels read from NCHW rows (the direct first-layer kernel): stateless call and
    plan, NCHW and channels-last outputs, a strided view as input, both bias modes, fused Relu,
    ONNX rounding."""
    N, C, H, W, OC, KH, KW, stride, pad = case
    rng = np.random.default_rng(51)
    x = rand_q(rng, (N, C, H, W), xdt)
    w = rng.integers(-127, 128, size=(OC, C, KH, KW)).astype(np.int8)
    ws = rng.uniform(0.002, 0.02, size=OC).astype(np.float32)
    wz = np.zeros(OC, np.int8)
    bias = rng.integers(-2000, 2001, size=OC).astype(np.int32)
    xz = 103 if xdt == np.uint8 else -9
    ys = np.float32(0.02 * 0.01 * 74 * 74 * np.sqrt(C * KH * KW) / 40)
    kw = dict(strides=(stride, stride), pads=(pad, pad))
    for bias_mode, flags in ((oracle.BIAS_ONNX_INT32, g.capi.BIAS_ONNX_INT32), (oracle.BIAS_REFERENCE_FLOAT, 0)):
        want = oracle.qlinear_conv_int(x, 0.02, xz, w, ws, wz, ys, 121, np.uint8, bias=bias, bias_mode=bias_mode, **kw)
        assert want.min() < want.max()
        got = g.ops.QLinearConv(g.dev(x), 0.02, xz, g.dev(w), g.dev(ws), g.dev(wz), ys, 121, g.dev(bias), flags=flags, **kw)
        np.testing.assert_array_equal(g.host(got), want)
        plan = g.ops.QLinearConvPlan(g.dev(w), g.dev(ws), g.dev(wz), g.dev(bias), **kw)
        out_cl = torch.empty((want.shape[0], want.shape[2], want.shape[3], want.shape[1]), dtype=torch.uint8,
                             device="cuda").permute(0, 3, 1, 2)
        out_nchw = torch.empty(want.shape, dtype=torch.uint8, device="cuda")
        # a view into a larger tensor: channel and image strides that are not the dense ones
        big = torch.zeros((N, C + 1, H + 2, W), dtype=g.dev(x).dtype, device="cuda")
        big[:, :C, 1:H + 1, :] = g.dev(x)
        view = big[:, :C, 1:H + 1, :]
        for xin in (g.dev(x), view):
            for out in (out_cl, out_nchw):
                out.zero_()
                plan.run(xin, 0.02, xz, ys, 121, flags=flags, out=out)
                np.testing.assert_array_equal(g.host(out), want)
        plan.close()
    fl = g.capi.BIAS_ONNX_INT32 | g.capi.FUSE_RELU | g.capi.ROUND_ONNX_RNE
    want = np.maximum(oracle.qlinear_conv_int(x, 0.02, xz, w, ws, wz, ys, -5, np.int8, bias=bias, bias_mode=oracle.BIAS_ONNX_INT32,
                                              round_mode=oracle.ROUND_ONNX_RNE, **kw), -5).astype(np.int8)
    got = g.ops.QLinearConv(g.dev(x), 0.02, xz, g.dev(w), g.dev(ws), g.dev(wz), ys, -5, g.dev(bias),
                            zero_point_dtype=torch.int8, flags=fl, **kw)
    np.testing.assert_array_equal(g.host(got), want)


@pytest.mark.parametrize("case", [
    # N, C, H, W, OC, K, stride, pad, group: the matrix-core kernel, the first-layer kernel, the depthwise kernel
    (2, 64, 9, 10, 96, 1, 1, 0, 1), (1, 32, 8, 8, 40, 3, 1, 1, 1), (2, 3, 20, 22, 32, 3, 2, 1, 1), (1, 48, 14, 6, 48, 3, 1, 1, 48)])
def test_qlinear_conv_with_output_zero_point_zero(g, oracle, case):
    """uint8 results with y_zero_point = 0 (every activation behind a Relu): the kernels leave the
    addition of the zero point out; negative values must saturate to 0 as the reference's clip does."""
    N, C, H, W, OC, K, stride, pad, group = case
    rng = np.random.default_rng(71)
    x = rand_q(rng, (N, C, H, W), np.uint8)
    w = rng.integers(-127, 128, size=(OC, C // group, K, K)).astype(np.int8)
    ws = rng.uniform(0.002, 0.02, size=OC).astype(np.float32)
    wz = np.zeros(OC, np.int8)
    bias = rng.integers(-300, 301, size=OC).astype(np.int32)
    ys = np.float32(0.02 * 0.01 * 74 * 74 * np.sqrt(C // group * K * K) / 60)
    kw = dict(strides=(stride, stride), pads=(pad, pad), group=group)
    for bias_mode, flags in ((oracle.BIAS_ONNX_INT32, g.capi.BIAS_ONNX_INT32), (oracle.BIAS_REFERENCE_FLOAT, 0)):
        want = oracle.qlinear_conv_int(x, 0.02, 101, w, ws, wz, ys, 0, np.uint8, bias=bias, bias_mode=bias_mode, **kw)
        assert (want == 0).mean() > 0.2 and want.max() > 100
        for xd in ((g.dev(x),) if C == 3 else (g.to_channels_last(g.dev(x)),)):
            for fl in (flags, flags | g.capi.FUSE_RELU):   # with a zero point of 0 the Relu changes nothing
                got = g.ops.QLinearConv(xd, 0.02, 101, g.dev(w), g.dev(ws), g.dev(wz), ys, 0, g.dev(bias), flags=fl, **kw)
                np.testing.assert_array_equal(g.host(got), want)


def _residual_sum(oracle, c, c_scale, c_zp, r, r_scale, r_zp, relu, out_scale, out_zp, out_dtype):
    """QuantizeLinear(act(DequantizeLinear(c) + DequantizeLinear(r))), op by op on the CPU."""
    s = oracle.binary(oracle.ADD, oracle.dequantize_linear(c, c_scale, c_zp), oracle.dequantize_linear(r, r_scale, r_zp))
    if relu:
        s = oracle.relu(s)
    return oracle.quantize_linear(s, out_scale, out_zp, out_dtype)


@pytest.mark.parametrize("ydt,rdt,odt", [(np.uint8, np.uint8, np.uint8), (np.int8, np.uint8, np.int8), (np.uint8, np.int8, np.uint8)])
@pytest.mark.parametrize("case", [
    # N, C, H, W, OC, K, stride, pad
    (2, 64, 9, 10, 256, 1, 1, 0), (1, 32, 7, 7, 24, 1, 1, 0), (2, 16, 8, 8, 70, 3, 1, 1), (1, 128, 6, 5, 128, 1, 2, 0)])
@pytest.mark.parametrize("form", ["searched", "exact"])
def test_qlinear_conv_with_fused_residual_sum(g, oracle, case, ydt, rdt, odt, form, monkeypatch):
    """chx_hip_qconv_plan_run_add against QLinearConv followed by the element-wise group, each on
    the CPU oracle: with and without Relu, all type combinations, channel counts that leave partial
    16-byte chunks, a residual with a padded pixel pitch.  Once as the library runs it by default (a
    uint8 sum in its two-multiply-add form wherever the plan's search finds constants that make it exact)
    and once with the operation-by-operation arithmetic forced."""
    if form == "exact":
        monkeypatch.setenv("CHX_HIP_AFFINE_RESIDUAL", "0")
    N, C, H, W, OC, K, stride, pad = case
    rng = np.random.default_rng(61)
    x = rand_q(rng, (N, C, H, W), np.uint8)
    w = rng.integers(-127, 128, size=(OC, C, K, K)).astype(np.int8)
    ws = rng.uniform(0.002, 0.02, size=OC).astype(np.float32)
    wz = np.zeros(OC, np.int8)
    bias = rng.integers(-500, 501, size=OC).astype(np.int32)
    ys = np.float32(0.02 * 0.01 * 74 * 74 * np.sqrt(C * K * K) / 40)
    yz = 119 if ydt == np.uint8 else -7
    kw = dict(strides=(stride, stride), pads=(pad, pad))
    conv = oracle.qlinear_conv_int(x, 0.02, 101, w, ws, wz, ys, yz, ydt, bias=bias, bias_mode=oracle.BIAS_ONNX_INT32, **kw)
    r = rand_q(rng, conv.shape, rdt)
    rs, rz = np.float32(0.037), (131 if rdt == np.uint8 else 5)
    os_, oz = np.float32(0.061), (99 if odt == np.uint8 else -20)
    plan = g.ops.QLinearConvPlan(g.dev(w), g.dev(ws), g.dev(wz), g.dev(bias), **kw)
    xd = g.to_channels_last(g.dev(x))
    n, oc, oh, ow = conv.shape
    pitch = (oc + 15) // 16 * 16
    r_padded = torch.zeros((n, oh, ow, pitch), dtype=g.dev(r).dtype, device="cuda")[..., :oc].permute(0, 3, 1, 2)
    r_padded.copy_(g.dev(r))
    for relu in (False, True):
        want = _residual_sum(oracle, conv, ys, yz, r, rs, rz, relu, os_, oz, odt)
        assert want.min() < want.max()
        for rd in (g.to_channels_last(g.dev(r)), r_padded):
            got = plan.run_add(xd, 0.02, 101, ys, yz, rd, rs, rz, os_, oz, relu, zero_point_dtype=TDT[ydt],
                               flags=g.capi.BIAS_ONNX_INT32, out=torch.zeros_like(rd, dtype=TDT[odt]))
            np.testing.assert_array_equal(g.host(got), want)
    # zero points of 0 on the residual and on the result (what lies between the Relu outputs of a
    # residual network): the kernel leaves out the two additions of 0 and, for uint8, the Relu,
    # which the saturation at 0 already is; negative sums must still come out as 0
    if rdt == np.uint8:
        for relu in (False, True):
            want = _residual_sum(oracle, conv, ys, yz, r, rs, 0, relu, os_, 0, odt)
            got = plan.run_add(xd, 0.02, 101, ys, yz, g.to_channels_last(g.dev(r)), rs, 0, os_, 0, relu, zero_point_dtype=TDT[ydt],
                               flags=g.capi.BIAS_ONNX_INT32, out=torch.zeros_like(g.to_channels_last(g.dev(r)), dtype=TDT[odt]))
            np.testing.assert_array_equal(g.host(got), want)
            assert want.min() < want.max()
    # which arithmetic the last sum used is on record; an int8 sum always keeps the long form
    forms = [l for l in plan.describe() if l.startswith("residual=")]
    if form == "exact":
        assert forms == []                    # no search was made
    else:
        assert forms and forms[-1] in ("residual=affine", "residual=exact")
        if odt == np.int8:
            assert forms[-1] == "residual=exact"
    # a caller that alternates between sets of parameters gets each one's own arithmetic back (the plan keeps what
    # it found for several of them): the first set again, after the others
    want = _residual_sum(oracle, conv, ys, yz, r, rs, rz, False, os_, oz, odt)
    rd = g.to_channels_last(g.dev(r))
    for _ in range(2):
        got = plan.run_add(xd, 0.02, 101, ys, yz, rd, rs, rz, os_, oz, False, zero_point_dtype=TDT[ydt],
                           flags=g.capi.BIAS_ONNX_INT32, out=torch.zeros_like(rd, dtype=TDT[odt]))
        np.testing.assert_array_equal(g.host(got), want)
    # operands that are not channels-last are refused, not converted
    with pytest.raises(g.capi.ChxHipError) as e:
        plan.run_add(xd, 0.02, 101, ys, yz, g.dev(r), rs, rz, os_, oz, True, zero_point_dtype=TDT[ydt],
                     flags=g.capi.BIAS_ONNX_INT32, out=torch.zeros(conv.shape, dtype=TDT[odt], device="cuda"))
    assert e.value.code == g.capi.EUNSUPPORTED
    # the sum written over its own residual operand (same type) is refused: the kernel may run more than once
    if rdt == odt:
        rd = g.to_channels_last(g.dev(r))
        with pytest.raises(g.capi.ChxHipError) as e:
            plan.run_add(xd, 0.02, 101, ys, yz, rd, rs, rz, os_, oz, True, zero_point_dtype=TDT[ydt], flags=g.capi.BIAS_ONNX_INT32, out=rd)
        assert e.value.code == g.capi.EINVAL and "overlaps" in str(e.value)
    plan.close()


def test_residual_sum_in_two_multiply_adds_over_all_code_pairs(g, oracle):
    """The short form of the fused sum, for the quantization parameters of the sixteen residual blocks of the
    ResNet-50 benchmark network (as calibrated: scales from 0.13 to 750, convolution zero points around 130) and a
    few others: a 1x1 convolution with identity weights passes every code c through, so one call per parameter set
    puts all 65536 (c, r) pairs through the kernel's epilogue, compared with the oracle's three ops.  The plan must
    find constants for most of them (the search is exhaustive over the pairs, so a found form is exact by
    construction; this test checks that through the kernel, and that the search is not vacuous)."""
    params = [(0.21131895, 122, 0.1626821, 130, 0.12926471, 0), (0.3873351, 147, 0.12926471, 0, 0.18676299, 0),
              (0.8456785, 137, 0.754098, 123, 0.51624763, 0), (1.5676626, 134, 0.51624763, 0, 1.0724535, 0),
              (14.470264, 128, 4.5852566, 0, 7.2227073, 0), (272.5226, 138, 273.2742, 117, 164.99017, 0),
              (746.74634, 141, 256.19128, 0, 383.77518, 0), (0.05, 120, 0.03, 7, 0.04, 33), (0.011, 0, 0.5, 255, 0.07, 250),
              (1.0, 128, 1.0, 128, 1.0, 0), (0.3, 3, 0.3, 3, 0.1, 0)]
    # x: 256 pixels x 256 channels, pixel p holds code p in every channel... the convolution must reproduce c exactly:
    # identity weights with scale 1, x_scale = y_scale, equal zero points -> y code == x code
    C = 64
    w = np.zeros((C, C, 1, 1), np.int8)
    w[np.arange(C), np.arange(C), 0, 0] = 1
    ws, wz = np.ones(C, np.float32), np.zeros(C, np.int8)
    codes = np.arange(256, dtype=np.uint8)
    x = np.broadcast_to(codes.reshape(1, 1, 256, 1), (1, C, 256, 256 // 1)).copy()      # c varies along H
    r = np.broadcast_to(codes.reshape(1, 1, 1, 256), (1, C, 256, 256)).copy()           # r varies along W
    found = 0
    for cs, cz, rs, rz, os_, oz in params:
        for relu in (True, False):
            plan = g.ops.QLinearConvPlan(g.dev(w), g.dev(ws), g.dev(wz), None)
            xd, rd = g.to_channels_last(g.dev(x)), g.to_channels_last(g.dev(r))
            conv = oracle.qlinear_conv_int(x, np.float32(cs), cz, w, ws, wz, np.float32(cs), cz, np.uint8)
            np.testing.assert_array_equal(conv, x)
            want = _residual_sum(oracle, conv, np.float32(cs), cz, r, np.float32(rs), rz, relu, np.float32(os_), oz, np.uint8)
            got = plan.run_add(xd, cs, cz, cs, cz, rd, rs, rz, os_, oz, relu, zero_point_dtype=torch.uint8, out=torch.zeros_like(rd))
            np.testing.assert_array_equal(g.host(got), want, err_msg=str((cs, cz, rs, rz, os_, oz, relu)))
            found += "residual=affine" in plan.describe()
            plan.close()
    assert found >= len(params)       # of 2 * len(params) sums


@pytest.mark.parametrize("tile", [(128, 128, 4), (64, 128, 4), (128, 64, 4), (64, 64, 4), (128, 128, 8), (128, 256, 8), (64, 128, 8)])
def test_every_launch_configuration_of_the_matrix_core_kernel(g, oracle, tile):
    """The tuner picks one of 4 tile shapes x 3 occupancy caps with four wavefronts per work-group, or
    one of 3 tile shapes with eight, per layer shape by timing, so a test that leaves the choice to it
    covers one configuration per case.  CHX_HIP_TILE forces each in turn: ragged pixel and channel
    tiles, 64- and 128-byte K steps (a configuration that exists for 128-byte steps only falls back to
    the tuner's choice on the others), padded and padding-free taps, channel counts that do not fill a
    K step, int32 results, the fused residual sum, work-groups that walk over several pixel tiles."""
    import os
    rng = np.random.default_rng(83)

    def qconv_case(N, C, H, W, OC, K, stride, pad):
        x = rand_q(rng, (N, C, H, W), np.uint8)
        w = rng.integers(-127, 128, size=(OC, C, K, K)).astype(np.int8)
        ws = rng.uniform(0.002, 0.02, size=OC).astype(np.float32)
        bias = rng.integers(-500, 501, size=OC).astype(np.int32)
        ys = np.float32(0.02 * 0.01 * 74 * 74 * np.sqrt(C * K * K) / 40)
        kw = dict(strides=(stride, stride), pads=(pad, pad))
        want = oracle.qlinear_conv_int(x, 0.02, 101, w, ws, np.zeros(OC, np.int8), ys, 119, np.uint8, bias=bias,
                                       bias_mode=oracle.BIAS_ONNX_INT32, **kw)
        return x, w, ws, bias, ys, kw, want

    # the last case has more pixel tiles than resident work-groups: each work-group walks over several
    convs = [qconv_case(3, 64, 13, 11, 200, 3, 1, 1), qconv_case(2, 256, 9, 7, 136, 1, 1, 0), qconv_case(2, 24, 11, 10, 72, 3, 2, 1),
             qconv_case(16, 64, 80, 79, 64, 1, 1, 0)]
    xi = rand_q(rng, (2, 128, 9, 9), np.uint8)
    wi = rand_q(rng, (80, 128, 3, 3), np.int8)
    want_int = oracle.conv_integer(xi, wi, 77, None, strides=(1, 1), pads=(0, 0), group=1, auto_pad="")
    # residual sum behind the second case
    x1, w1, ws1, bias1, ys1, kw1, conv1 = convs[1]
    r = rand_q(rng, conv1.shape, np.uint8)
    want_sum = _residual_sum(oracle, conv1, ys1, 119, r, np.float32(0.037), 131, True, np.float32(0.061), 99, np.uint8)
    before = os.environ.get("CHX_HIP_TILE")
    try:
        for cap in ((0, 2, 1) if tile[2] == 4 else (0,)):
            os.environ["CHX_HIP_TILE"] = "%d,%d,%d,%d" % (tile[0], tile[1], cap, tile[2])
            for x, w, ws, bias, ys, kw, want in convs:
                plan = g.ops.QLinearConvPlan(g.dev(w), g.dev(ws), g.dev(np.zeros(len(ws), np.int8)), g.dev(bias), **kw)
                got = plan.run(g.to_channels_last(g.dev(x)), 0.02, 101, ys, 119, torch.uint8, flags=g.capi.BIAS_ONNX_INT32)
                np.testing.assert_array_equal(g.host(got), want, err_msg="tile %s cap %d conv %s" % (tile, cap, x.shape))
                if x is x1:
                    rd = g.to_channels_last(g.dev(r))
                    got = plan.run_add(g.to_channels_last(g.dev(x)), 0.02, 101, ys, 119, rd, 0.037, 131, 0.061, 99, True,
                                       zero_point_dtype=torch.uint8, flags=g.capi.BIAS_ONNX_INT32, out=torch.zeros_like(rd))
                    np.testing.assert_array_equal(g.host(got), want_sum, err_msg="tile %s cap %d residual sum" % (tile, cap))
                plan.close()
            got = g.ops.ConvInteger(g.to_channels_last(g.dev(xi)), g.dev(wi), 77, None)
            np.testing.assert_array_equal(g.host(got), want_int, err_msg="tile %s cap %d ConvInteger" % (tile, cap))
    finally:
        if before is None:
            os.environ.pop("CHX_HIP_TILE", None)
        else:
            os.environ["CHX_HIP_TILE"] = before


@pytest.mark.parametrize("case", [
    # N, C, H, W, OC1, OC2, K, stride, pad
    (2, 256, 14, 14, 128, 512, 1, 2, 0),    # a down-sampling block: main path and shortcut, stride 2
    (3, 64, 9, 11, 64, 256, 1, 1, 0),       # the first block: 64-channel tiles only, a 64-byte K step
    (1, 128, 7, 6, 192, 72, 3, 1, 1),       # padded taps, a ragged second half, a split that only 64-channel tiles divide
    (16, 64, 40, 41, 128, 128, 1, 1, 0)])   # more pixel tiles than resident work-groups
def test_two_convolutions_of_one_input_in_one_launch(g, oracle, case):
    """chx_hip_qconv_plan_run_pair against the two QLinearConv on the CPU oracle, each with its own output quantization
    (and one of them with a fused Relu): the tuner's choice and every launch configuration whose tile divides the split."""
    import os
    N, C, H, W, OC1, OC2, K, stride, pad = case
    rng = np.random.default_rng(97)
    x = rand_q(rng, (N, C, H, W), np.uint8)
    w = rng.integers(-127, 128, size=(OC1 + OC2, C, K, K)).astype(np.int8)
    ws = rng.uniform(0.002, 0.02, size=OC1 + OC2).astype(np.float32)
    wz = np.zeros(OC1 + OC2, np.int8)
    bias = rng.integers(-500, 501, size=OC1 + OC2).astype(np.int32)
    ys1 = np.float32(0.02 * 0.01 * 74 * 74 * np.sqrt(C * K * K) / 40)
    ys2 = np.float32(ys1 * 1.7)
    kw = dict(strides=(stride, stride), pads=(pad, pad))
    want1 = oracle.qlinear_conv_int(x, 0.02, 101, w[:OC1], ws[:OC1], wz[:OC1], ys1, 0, np.uint8, bias=bias[:OC1],
                                    bias_mode=oracle.BIAS_ONNX_INT32, **kw)
    want2 = oracle.qlinear_conv_int(x, 0.02, 101, w[OC1:], ws[OC1:], wz[OC1:], ys2, -9, np.int8, bias=bias[OC1:],
                                    bias_mode=oracle.BIAS_ONNX_INT32, **kw)
    assert want1.min() < want1.max() and want2.min() < want2.max()
    xd = g.to_channels_last(g.dev(x))
    flags = (g.capi.BIAS_ONNX_INT32 | g.capi.FUSE_RELU, g.capi.BIAS_ONNX_INT32)
    before = os.environ.get("CHX_HIP_TILE")
    try:
        for tile in (None, "128,128,0,4", "64,128,0,4", "128,64,2,4", "64,64,1,4", "128,128,0,8", "128,256,0,8", "64,128,0,8"):
            if tile is None:
                os.environ.pop("CHX_HIP_TILE", None)
            else:
                os.environ["CHX_HIP_TILE"] = tile       # a tile that does not divide the split falls back to 64 channels
            plan = g.ops.QLinearConvPlan(g.dev(w), g.dev(ws), g.dev(wz), g.dev(bias), **kw)
            for _ in range(2):
                got1, got2 = plan.run_pair(xd, 0.02, 101, OC1, ys1, 0, ys2, -9, zero_point_dtypes=(torch.uint8, torch.int8), flags=flags)
                np.testing.assert_array_equal(g.host(got1), want1, err_msg="tile %s first" % tile)
                np.testing.assert_array_equal(g.host(got2), want2, err_msg="tile %s second" % tile)
            plan.close()
    finally:
        if before is None:
            os.environ.pop("CHX_HIP_TILE", None)
        else:
            os.environ["CHX_HIP_TILE"] = before
    # what the entry point refuses
    plan = g.ops.QLinearConvPlan(g.dev(w), g.dev(ws), g.dev(wz), g.dev(bias), **kw)
    with pytest.raises(g.capi.ChxHipError) as e:
        plan.run_pair(xd, 0.02, 101, OC1 - 32, ys1, 0, ys2, -9, zero_point_dtypes=(torch.uint8, torch.int8), flags=flags)          # not a multiple of 64
    assert e.value.code == g.capi.EUNSUPPORTED
    with pytest.raises(g.capi.ChxHipError) as e:
        plan.run_pair(xd, 0.02, 101, OC1, ys1, 0, ys2, -9, zero_point_dtypes=(torch.uint8, torch.int8), flags=(g.capi.BIAS_ONNX_INT32, 0))    # the halves differ in the bias mode
    assert e.value.code == g.capi.EINVAL
    with pytest.raises(g.capi.ChxHipError) as e:
        plan.run_pair(g.dev(x), 0.02, 101, OC1, ys1, 0, ys2, -9, zero_point_dtypes=(torch.uint8, torch.int8), flags=flags)          # NCHW operands are not converted
    assert e.value.code == g.capi.EUNSUPPORTED
    plan.close()


def test_results_stored_minus_128(g, oracle):
    """CHX_HIP_STORE_MINUS_128: a uint8 result stored as code - 128 in an int8 array is the same tensor as an int8 one
    with zero point zp - 128.  The flag on the three plan entry points gives the bytes of the plain result with the top
    bit flipped, and a convolution (or a fused residual sum) that reads such an array as int8 gives the bytes it gives
    on the uint8 array: a chain of two convolutions with a residual sum, every intermediate in both storages."""
    rng = np.random.default_rng(151)
    N, C, H, W, OC = 2, 64, 9, 10, 128
    x = rand_q(rng, (N, C, H, W), np.uint8)
    w1 = rng.integers(-127, 128, size=(OC, C, 3, 3)).astype(np.int8)
    w2 = rng.integers(-127, 128, size=(C, OC, 1, 1)).astype(np.int8)
    ws1, ws2 = rng.uniform(0.002, 0.02, size=OC).astype(np.float32), rng.uniform(0.002, 0.02, size=C).astype(np.float32)
    b1, b2 = rng.integers(-500, 501, size=OC).astype(np.int32), rng.integers(-500, 501, size=C).astype(np.int32)
    y1s, y1z = np.float32(0.02 * 0.01 * 74 * 74 * np.sqrt(C * 9) / 40), 17
    y2s, y2z = np.float32(y1s * 0.01 * 74 * np.sqrt(OC) / 3), 119
    os_, oz = np.float32(0.05), 0
    kw1 = dict(strides=(1, 1), pads=(1, 1))
    a = oracle.qlinear_conv_int(x, 0.02, 101, w1, ws1, np.zeros(OC, np.int8), y1s, y1z, np.uint8, bias=b1, bias_mode=oracle.BIAS_ONNX_INT32, **kw1)
    c = oracle.qlinear_conv_int(a, y1s, y1z, w2, ws2, np.zeros(C, np.int8), y2s, y2z, np.uint8, bias=b2, bias_mode=oracle.BIAS_ONNX_INT32)
    for relu in (True, False):
        want_sum = _residual_sum(oracle, c, y2s, y2z, x, np.float32(0.02), 101, relu, os_, oz, np.uint8)
        assert a.min() < a.max() and c.min() < c.max() and want_sum.min() < want_sum.max()
        flip = lambda t: (t.view(torch.uint8) ^ 0x80)       # int8 storage -> the uint8 codes it stands for
        F = g.capi.BIAS_ONNX_INT32
        S = F | g.capi.STORE_MINUS_128
        p1 = g.ops.QLinearConvPlan(g.dev(w1), g.dev(ws1), g.dev(np.zeros(OC, np.int8)), g.dev(b1), **kw1)
        p2 = g.ops.QLinearConvPlan(g.dev(w2), g.dev(ws2), g.dev(np.zeros(C, np.int8)), g.dev(b2))
        xd = g.to_channels_last(g.dev(x))
        xs = (xd.view(torch.uint8) ^ 0x80).view(torch.int8)        # the input stored minus 128
        for x_in, x_zp in ((xd, 101), (xs, 101 - 128)):
            # first convolution, result in either storage
            a_u = p1.run(x_in, 0.02, x_zp, y1s, y1z, torch.uint8, flags=F)
            a_s = p1.run(x_in, 0.02, x_zp, y1s, y1z, torch.int8, flags=S)
            np.testing.assert_array_equal(g.host(a_u), a)
            assert a_s.dtype == torch.int8
            np.testing.assert_array_equal(g.host(flip(a_s)), a)
            for a_in, a_zp in ((a_u, y1z), (a_s, y1z - 128)):
                # second convolution with the block's residual sum (the residual in either storage too), result in either storage
                for r_in, r_zp in ((xd, 101), (xs, 101 - 128)):
                    got = p2.run_add(a_in, y1s, a_zp, y2s, y2z, r_in, 0.02, r_zp, os_, oz, relu, zero_point_dtype=torch.uint8, flags=F,
                                     out=torch.zeros_like(xd))
                    np.testing.assert_array_equal(g.host(got), want_sum)
                    got = p2.run_add(a_in, y1s, a_zp, y2s, y2z, r_in, 0.02, r_zp, os_, oz, relu, zero_point_dtype=torch.uint8, flags=S,
                                     out=torch.zeros_like(xs))
                    np.testing.assert_array_equal(g.host(flip(got)), want_sum)
        # two convolutions in one launch, one result in each storage
        wp = np.concatenate([w1, w1[::-1]])
        pp = g.ops.QLinearConvPlan(g.dev(wp), g.dev(np.concatenate([ws1, ws1[::-1]])), g.dev(np.zeros(2 * OC, np.int8)), g.dev(np.concatenate([b1, b1[::-1]])), **kw1)
        a_rev = oracle.qlinear_conv_int(x, 0.02, 101, w1[::-1].copy(), ws1[::-1].copy(), np.zeros(OC, np.int8), y1s, 33, np.uint8, bias=b1[::-1].copy(),
                                        bias_mode=oracle.BIAS_ONNX_INT32, **kw1)
        o1, o2 = pp.run_pair(xs, 0.02, 101 - 128, OC, y1s, y1z, y1s, 33, zero_point_dtypes=(torch.int8, torch.uint8), flags=(S, F))
        np.testing.assert_array_equal(g.host(flip(o1)), a)
        np.testing.assert_array_equal(g.host(o2), a_rev)
        o1, o2 = pp.run_pair(xd, 0.02, 101, OC, y1s, y1z, y1s, 33, zero_point_dtypes=(torch.uint8, torch.int8), flags=(F, S))
        np.testing.assert_array_equal(g.host(o1), a)
        np.testing.assert_array_equal(g.host(flip(o2)), a_rev)
        # the flag wants an int8 array, and a kernel that can honour it
        with pytest.raises(g.capi.ChxHipError) as e:
            p1.run(xd, 0.02, 101, y1s, y1z, torch.uint8, flags=S)
        assert e.value.code == g.capi.EINVAL
        with pytest.raises(g.capi.ChxHipError) as e:
            p1.run(g.dev(x), 0.02, 101, y1s, y1z, torch.int8, flags=S)        # NCHW: the result would be transposed afterwards
        assert e.value.code == g.capi.EUNSUPPORTED
        for p in (p1, p2, pp):
            p.close()
        # the depthwise 3x3 kernel stores the codes minus 128 as well; a grouped convolution of another shape does not
        Cd = 32
        xdw = rand_q(rng, (2, Cd, 9, 10), np.uint8)
        wdw = rng.integers(-127, 128, size=(Cd, 1, 3, 3)).astype(np.int8)
        wsd = rng.uniform(0.002, 0.02, size=Cd).astype(np.float32)
        bd = rng.integers(-500, 501, size=Cd).astype(np.int32)
        yds = np.float32(0.02 * 0.01 * 74 * 74 * 3 / 40)
        kwd = dict(strides=(1, 1), pads=(1, 1), group=Cd)
        want_dw = oracle.qlinear_conv_int(xdw, 0.02, 101, wdw, wsd, np.zeros(Cd, np.int8), yds, 119, np.uint8, bias=bd,
                                          bias_mode=oracle.BIAS_ONNX_INT32, **kwd)
        pd = g.ops.QLinearConvPlan(g.dev(wdw), g.dev(wsd), g.dev(np.zeros(Cd, np.int8)), g.dev(bd), **kwd)
        xdd = g.to_channels_last(g.dev(xdw))
        np.testing.assert_array_equal(g.host(pd.run(xdd, 0.02, 101, yds, 119, torch.uint8, flags=F)), want_dw)
        np.testing.assert_array_equal(g.host(flip(pd.run(xdd, 0.02, 101, yds, 119, torch.int8, flags=S))), want_dw)
        np.testing.assert_array_equal(g.host(flip(pd.run(g.ops.codes_minus_128(xdd), 0.02, 101 - 128, yds, 119, torch.int8, flags=S))), want_dw)
        pd.close()
        wg = rng.integers(-127, 128, size=(Cd, 2, 3, 3)).astype(np.int8)
        pg = g.ops.QLinearConvPlan(g.dev(wg), g.dev(wsd), g.dev(np.zeros(Cd, np.int8)), g.dev(bd), strides=(1, 1), pads=(1, 1), group=Cd // 2)
        with pytest.raises(g.capi.ChxHipError) as e:
            pg.run(xdd, 0.02, 101, yds, 119, torch.int8, flags=S)
        assert e.value.code == g.capi.EUNSUPPORTED
        pg.close()


def test_random_convolution_sweep(g, oracle):
    """Seeded random QLinearConv / ConvInteger configurations across every dispatch path (matrix-core
    tiles, first-layer kernel, depthwise kernel, generic kernel): shapes, kernel sizes, strides, pads,
    groups, element types, layouts, bias modes, per-tensor and per-channel scales; bit-exact."""
    rng = np.random.default_rng(2024)
    seen = 0
    for trial in range(70):
        kh, kw = (int(rng.choice([1, 2, 3, 5, 7])) for _ in range(2))
        kind = trial % 5
        if kind == 0:        # depthwise 3x3 and its neighbours
            C = int(rng.integers(1, 80))
            group, OC = C, C * int(rng.choice([1, 1, 1, 2]))
            kh = kw = int(rng.choice([3, 3, 1, 5]))
            if trial % 10 == 0:      # every other one in the form the depthwise kernel takes: channels in sixteens, 3x3
                C = group = OC = 16 * int(rng.integers(1, 7))
                kh = kw = 3
        elif kind == 1:      # grouped
            group = int(rng.choice([2, 3, 4]))
            C, OC = group * int(rng.integers(1, 20)), group * int(rng.integers(1, 20))
        elif kind == 2:      # few planar channels (first layer)
            group, C, OC = 1, int(rng.integers(1, 5)), int(rng.integers(1, 70))
        else:                # dense
            group, C, OC = 1, int(rng.choice([8, 16, 24, 32, 48, 64, 72, 128, 160, 256, int(rng.integers(1, 200))])), int(rng.integers(1, 200))
        H, W = int(rng.integers(1, 22)), int(rng.integers(1, 22))
        sh, sw = int(rng.choice([1, 1, 2, 3])), int(rng.choice([1, 1, 2, 3]))
        ph, pw = int(rng.integers(0, kh // 2 + 2)), int(rng.integers(0, kw // 2 + 2))
        if H + 2 * ph < kh or W + 2 * pw < kw:
            continue
        N = int(rng.integers(1, 4))
        xdt = [np.uint8, np.int8][int(rng.integers(0, 2))]
        wdt = [np.int8, np.int8, np.uint8][int(rng.integers(0, 3))]
        if kind == 0 and trial % 10 == 0:
            wdt = np.int8
        ydt = [np.uint8, np.int8][int(rng.integers(0, 2))]
        x = rand_q(rng, (N, C, H, W), xdt)
        w = rand_q(rng, (OC, C // group, kh, kw), wdt)
        per_channel = bool(rng.integers(0, 2))
        ws = rng.uniform(0.002, 0.02, size=OC if per_channel else 1).astype(np.float32)
        wz = rand_q(rng, (OC if per_channel else 1,), wdt) if rng.integers(0, 3) == 0 else np.zeros(OC if per_channel else 1, wdt)
        xz = int(rand_q(rng, (1,), xdt)[0])
        yz = int(rand_q(rng, (1,), ydt)[0]) if rng.integers(0, 4) else 0
        K = (C // group) * kh * kw
        ys = np.float32(0.02 * 0.01 * 74 * 74 * np.sqrt(K) / float(rng.choice([20, 60, 200])))
        bias_mode = int(rng.integers(0, 3))
        bias = rng.integers(-400, 401, size=OC).astype(np.int32)
        kw_ = dict(strides=(sh, sw), pads=(ph, pw), group=group)
        okw, flags, b = dict(kw_), 0, None
        if bias_mode == 1:
            b, okw["bias"], okw["bias_mode"] = bias, bias, oracle.BIAS_REFERENCE_FLOAT
        elif bias_mode == 2:
            b, okw["bias"], okw["bias_mode"], flags = bias, bias, oracle.BIAS_ONNX_INT32, g.capi.BIAS_ONNX_INT32
        tag = "trial %d: x%s %s w%s %s strides %s pads %s group %d per_channel %s bias %d y %s" % (
            trial, x.shape, xdt.__name__, w.shape, wdt.__name__, (sh, sw), (ph, pw), group, per_channel, bias_mode, ydt.__name__)
        xd = g.dev(x) if rng.integers(0, 2) and not (kind == 0 and trial % 10 == 0) else g.to_channels_last(g.dev(x))
        wsd, wzd = (g.dev(ws), g.dev(wz)) if per_channel else (g.dev(ws.reshape(())), g.dev(wz.reshape(())))
        want = oracle.qlinear_conv_int(x, 0.02, xz, w, ws if per_channel else ws[:1], wz if per_channel else wz[:1], ys, yz, ydt, **okw)
        got = g.ops.QLinearConv(xd, 0.02, xz, g.dev(w), wsd, wzd, ys, yz, None if b is None else g.dev(b),
                                zero_point_dtype=TDT[ydt], flags=flags, **kw_)
        np.testing.assert_array_equal(g.host(got), want, err_msg=tag)
        want_i = oracle.conv_integer(x, w, xz, wz if per_channel else wz[:1], auto_pad="", **kw_)
        got_i = g.ops.ConvInteger(xd, g.dev(w), xz, wzd if per_channel else g.dev(wz[:1].reshape(())), **kw_)
        np.testing.assert_array_equal(g.host(got_i), want_i, err_msg=tag)
        seen += 1
    assert seen >= 55


def test_random_matmul_sweep(g, oracle):
    """Seeded random MatMulInteger / QLinearMatMul shapes (2-D, batched N-D, K and N that leave
    partial tiles, every element-type pairing, zero points, strided operands); bit-exact."""
    rng = np.random.default_rng(4242)
    for trial in range(40):
        M, K, N = (int(rng.choice([1, 2, 7, 16, 33, 64, 100, 129, int(rng.integers(1, 300))])) for _ in range(3))
        batch = [(), (), (3,), (2, 2)][int(rng.integers(0, 4))]
        adt = [np.uint8, np.int8][int(rng.integers(0, 2))]
        bdt = [np.int8, np.uint8][int(rng.integers(0, 2))]
        a, b = rand_q(rng, batch + (M, K), adt), rand_q(rng, batch + (K, N), bdt)
        az = rand_q(rng, (1,), adt) if rng.integers(0, 2) else None
        bz = rand_q(rng, (N,) if rng.integers(0, 2) else (1,), bdt) if rng.integers(0, 2) else None
        tag = "trial %d: a%s %s b%s %s" % (trial, a.shape, adt.__name__, b.shape, bdt.__name__)
        bd = g.dev(b) if rng.integers(0, 2) else g.dev(np.ascontiguousarray(np.swapaxes(b, -1, -2))).transpose(-1, -2)
        got = g.ops.MatMulInteger(g.dev(a), bd, None if az is None else g.dev(az), None if bz is None else g.dev(bz))
        np.testing.assert_array_equal(g.host(got), oracle.matmul_integer(a, b, az, bz), err_msg=tag)
        ydt = [np.uint8, np.int8][int(rng.integers(0, 2))]
        a_zp, b_zp, y_zp = int(rand_q(rng, (1,), adt)[0]), int(rand_q(rng, (1,), bdt)[0]), int(rand_q(rng, (1,), ydt)[0])
        b_scale = np.float32(rng.uniform(0.002, 0.02))
        y_scale = np.float32(0.02 * 0.01 * 74 * 74 * np.sqrt(K) / float(rng.choice([20, 60, 200])))
        want = oracle.qlinear_matmul_int(a, 0.02, a_zp, b, b_scale, b_zp, y_scale, y_zp, ydt)
        got = g.ops.QLinearMatMul(g.dev(a), 0.02, a_zp, bd, b_scale, b_zp, y_scale, y_zp, zero_point_dtype=TDT[ydt])
        np.testing.assert_array_equal(g.host(got), want, err_msg=tag + " QLinearMatMul -> " + ydt.__name__)


def _depth_folded(x, w, zp, sd, pd_b, pd_e, od):
    """The 2-D problem that output depth `od` of a 3-D convolution is: the KD input slices under the window stacked
    along the channels (channel c, tap kd -> c*KD + kd, so groups stay contiguous), depth padding filled with the zero
    point (x - zero_point = 0 there: the reference's zero padding of the zero-point-subtracted tensor)."""
    n, c, d, h, wd = x.shape
    kd = w.shape[2]
    xp = np.full((n, c, d + pd_b + pd_e, h, wd), zp, x.dtype)
    xp[:, :, pd_b:pd_b + d] = x
    x2 = xp[:, :, od * sd:od * sd + kd].reshape(n, c * kd, h, wd)
    w2 = w.reshape(w.shape[0], w.shape[1] * kd, w.shape[3], w.shape[4])
    return np.ascontiguousarray(x2), np.ascontiguousarray(w2)


def test_convolutions_over_one_and_three_spatial_axes(g, oracle):
    """ComplementStride / ComplementPad / GroupedConv are rank-generic (runtime/chainerx_util.cc:180-200,313-340): x [N,C,L]
    against the 2-D oracle on images one pixel high; x [N,C,D,H,W] against the 2-D oracle on the depth-folded problem."""
    rng = np.random.default_rng(61)
    # one spatial axis: reaches the matrix-core kernel (64 channels) and the direct kernel (groups)
    for c, oc, group in ((64, 32, 1), (12, 8, 2)):
        x, w = rand_q(rng, (3, c, 50), np.uint8), rand_q(rng, (oc, c // group, 5), np.int8)
        ws, wz = rng.uniform(0.001, 0.01, oc).astype(np.float32), np.zeros(oc, np.int8)
        bias = rng.integers(-500, 500, oc).astype(np.int32)
        got = g.ops.QLinearConv(g.dev(x), 0.02, 120, g.dev(w), g.dev(ws), g.dev(wz), 0.05, 128, g.dev(bias), strides=[2], pads=[2, 1],
                                group=group, flags=g.capi.BIAS_ONNX_INT32)
        want = oracle.qlinear_conv_int(x[:, :, None, :], 0.02, 120, w[:, :, None, :], ws, wz, 0.05, 128, np.uint8, bias=bias, strides=(1, 2),
                                       pads=(0, 2, 0, 1), group=group, bias_mode=oracle.BIAS_ONNX_INT32)
        assert tuple(got.shape) == (3, oc, want.shape[3])
        np.testing.assert_array_equal(g.host(got), want[:, :, 0, :])
        goti = g.ops.ConvInteger(g.dev(x), g.dev(w), 120, None, strides=[2], pads=[2, 1], group=group)
        np.testing.assert_array_equal(g.host(goti), oracle.conv_integer(x[:, :, None, :], w[:, :, None, :], 120, None, strides=(1, 2),
                                                                         pads=(0, 2, 0, 1), group=group)[:, :, 0, :])
    # three spatial axes
    for group in (1, 2):
        x, w = rand_q(rng, (2, 6, 7, 9, 8), np.uint8), rand_q(rng, (4, 6 // group, 3, 2, 3), np.int8)
        ws, wz = rng.uniform(0.001, 0.01, 4).astype(np.float32), rand_q(rng, (4,), np.int8)
        strides, pb, pe = (2, 1, 2), (1, 0, 2), (1, 1, 0)
        got = g.ops.QLinearConv(g.dev(x), 0.03, 7, g.dev(w), g.dev(ws), g.dev(wz), 0.04, 100, None, strides=list(strides),
                                pads=list(pb) + list(pe), group=group)
        goti = g.ops.ConvInteger(g.dev(x), g.dev(w), 7, g.dev(wz), strides=list(strides), pads=list(pb) + list(pe), group=group)
        od_n = (7 + pb[0] + pe[0] - 3) // strides[0] + 1
        assert got.shape[2] == od_n and goti.dtype == torch.int32
        for od in range(od_n):
            x2, w2 = _depth_folded(x, w, 7, strides[0], pb[0], pe[0], od)
            want = oracle.qlinear_conv_int(x2, 0.03, 7, w2, ws, wz, 0.04, 100, np.uint8, strides=strides[1:], pads=(pb[1], pb[2], pe[1], pe[2]),
                                           group=group, bias_mode=oracle.BIAS_REFERENCE_FLOAT)
            np.testing.assert_array_equal(g.host(got)[:, :, od], want, err_msg="group %d depth %d" % (group, od))
            wanti = oracle.conv_integer(x2, w2, 7, wz, strides=strides[1:], pads=(pb[1], pb[2], pe[1], pe[2]), group=group)
            np.testing.assert_array_equal(g.host(goti)[:, :, od], wanti)
    with pytest.raises(g.capi.ChxHipError):
        g.ops.ConvInteger(g.dev(rand_q(rng, (1, 2, 3, 3, 3, 3), np.uint8)), g.dev(rand_q(rng, (1, 2, 1, 1, 1, 1), np.int8)))


def test_codes_minus_128_both_ways(g):
    """chx_hip_codes_minus_128: uint8 -> int8 is code - 128, int8 -> uint8 code + 128, through any strides; other
    pairs of types and differing shapes are refused."""
    rng = np.random.default_rng(152)
    u = rng.integers(0, 256, size=(3, 5, 7, 16)).astype(np.uint8)
    want = (u.astype(np.int16) - 128).astype(np.int8)
    du = torch.from_numpy(u).cuda()
    s = g.ops.codes_minus_128(du)
    assert s.dtype == torch.int8
    np.testing.assert_array_equal(s.cpu().numpy(), want)
    np.testing.assert_array_equal(g.ops.codes_minus_128(s).cpu().numpy(), u)
    # channels-last source, dense destination; a sliced destination
    cl = du.permute(0, 3, 1, 2)
    np.testing.assert_array_equal(g.ops.codes_minus_128(cl.contiguous(memory_format=torch.channels_last)).cpu().numpy(), want.transpose(0, 3, 1, 2))
    wide = torch.zeros((3, 5, 7, 32), dtype=torch.int8, device="cuda")
    g.ops.codes_minus_128(du, out=wide[..., 8:24])
    np.testing.assert_array_equal(wide[..., 8:24].cpu().numpy(), want)
    assert not wide[..., :8].any() and not wide[..., 24:].any()
    assert g.ops.codes_minus_128(torch.empty((0, 4), dtype=torch.uint8, device="cuda")).shape == (0, 4)
    for bad_out in (torch.empty_like(du), torch.empty((3, 5, 7, 16), dtype=torch.int32, device="cuda"),
                    torch.empty((3, 5, 7, 8), dtype=torch.int8, device="cuda")):
        with pytest.raises(g.capi.ChxHipError):
            g.ops.codes_minus_128(du, out=bad_out)
