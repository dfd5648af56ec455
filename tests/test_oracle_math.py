"""Pins the CPU oracle where the ONNX vectors leave it open: against independent
numpy restatements (different code, different loop structure), closed forms and
invariants.  A dropped term, a wrong sign, a transposed operand or a wrong pad
side fails at least one test here."""
import numpy as np
import pytest


def np_quantize(x, scale, zp, lo, hi):
    """quantize_array (runtime/ops/quantize.cc:16-35) spelled in numpy fp32 ops."""
    s = x.astype(np.float32) / np.float32(scale)
    if zp != 0:
        s = s + np.float32(zp)
    s = np.maximum(np.float32(lo), np.minimum(s, np.float32(hi))) + np.float32(0.5)
    return np.trunc(s).astype(np.int64)


@pytest.mark.parametrize("dtype,zp,scale", [(np.uint8, 128, 0.02), (np.uint8, 0, 1.0 / 255), (np.int8, 0, 0.05),
                                            (np.int8, -7, 0.3), (np.uint8, 255, 3.0), (np.int8, 127, 1e-3)])
def test_quantize_vs_numpy(oracle, dtype, zp, scale):
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.standard_normal(20000).astype(np.float32) * 10,
                        np.array([0, -0.0, 1e-30, -1e-30, 1e30, -1e30, 0.5 * scale, 1.5 * scale, 2.5 * scale,
                                  -0.5 * scale, -1.5 * scale], np.float32),
                        (np.arange(-300, 300, dtype=np.float32) + 0.5) * np.float32(scale)])
    lo, hi = (0, 255) if dtype == np.uint8 else (-128, 127)
    got = oracle.quantize_linear(x, scale, zp, dtype)
    np.testing.assert_array_equal(got.astype(np.int64), np_quantize(x, scale, zp, lo, hi))
    # range + monotone non-decreasing in x
    order = np.argsort(x, kind="stable")
    assert np.all(np.diff(got[order].astype(np.int64)) >= 0)
    assert got.min() >= lo and got.max() <= hi


def test_quantize_int8_truncation_quirk(oracle):
    # +0.5f then a truncating cast rounds negative values toward zero-ish:
    # -1.7 -> -1.2 -> -1 (a round-to-nearest would give -2).  runtime/ops/quantize.cc:34.
    y = oracle.quantize_linear(np.array([-1.7, -1.2, -0.6, 1.7], np.float32), 1.0, 0, np.int8)
    assert y.tolist() == [-1, 0, 0, 2]
    y = oracle.quantize_linear(np.array([-1.7, 2.5, 3.5], np.float32), 1.0, 0, np.int8, round_mode=oracle.ROUND_ONNX_RNE)
    assert y.tolist() == [-2, 2, 4]
    # -128 is unreachable for int8 under the reference rule (clip to -128, +0.5, truncate -> -127)
    assert oracle.quantize_linear(np.array([-1e9], np.float32), 1.0, 0, np.int8).tolist() == [-127]


@pytest.mark.parametrize("dtype,zp", [(np.uint8, 0), (np.uint8, 128), (np.uint8, 255)])
@pytest.mark.parametrize("scale", [0.05, 1.0 / 255, 2.0, 0.00369204697])
def test_quantize_of_dequantize_is_identity(oracle, dtype, zp, scale):
    q = np.arange(0, 256).astype(dtype)
    x = oracle.dequantize_linear(q, scale, zp)
    np.testing.assert_array_equal(x, ((q.astype(np.float32) - np.float32(zp)) * np.float32(scale)))
    np.testing.assert_array_equal(oracle.quantize_linear(x, scale, zp, dtype), q)


def test_dequantize_exhaustive_int8(oracle):
    q = np.arange(-128, 128).astype(np.int8)
    for zp in (0, -5, 127):
        x = oracle.dequantize_linear(q, 0.1, zp)
        want = (q.astype(np.float64) - zp) * float(np.float32(0.1))
        np.testing.assert_array_equal(x, want.astype(np.float32))  # exact product fits? compare after fp32 rounding
        np.testing.assert_array_equal(x, oracle.dequantize_linear(q, 0.1, zp, multipass=True))


@pytest.mark.parametrize("adt,bdt", [(np.uint8, np.int8), (np.uint8, np.uint8), (np.int8, np.int8)])
def test_matmul_integer_vs_int64(oracle, adt, bdt):
    rng = np.random.default_rng(2)
    lo_a, hi_a = (0, 256) if adt == np.uint8 else (-128, 128)
    lo_b, hi_b = (0, 256) if bdt == np.uint8 else (-128, 128)
    a = rng.integers(lo_a, hi_a, size=(3, 5, 37)).astype(adt)
    b = rng.integers(lo_b, hi_b, size=(3, 37, 11)).astype(bdt)
    bz = rng.integers(lo_b, hi_b, size=11).astype(bdt)
    az = np.array([7]).astype(adt)
    want = np.einsum("bmk,bkn->bmn", a.astype(np.int64) - int(az[0]), b.astype(np.int64) - bz.astype(np.int64)[None, None, :])
    np.testing.assert_array_equal(oracle.matmul_integer(a, b, az, bz), want)
    np.testing.assert_array_equal(oracle.matmul_integer(a[0], b[0], None, None), a[0].astype(np.int64) @ b[0].astype(np.int64))



def np_conv_int64(x, w, strides, pads4, group):
    """Independent int64 convolution: explicit zero padding + window slicing."""
    N, C, H, W = x.shape
    OC, Cg, KH, KW = w.shape
    ph0, pw0, ph1, pw1 = pads4
    xp = np.zeros((N, C, H + ph0 + ph1, W + pw0 + pw1), np.int64)
    xp[:, :, ph0:ph0 + H, pw0:pw0 + W] = x
    OH = (H + ph0 + ph1 - KH) // strides[0] + 1
    OW = (W + pw0 + pw1 - KW) // strides[1] + 1
    y = np.zeros((N, OC, OH, OW), np.int64)
    OCg = OC // group
    for g in range(group):
        xs = xp[:, g * Cg:(g + 1) * Cg]
        ws = w[g * OCg:(g + 1) * OCg]
        for oh in range(OH):
            for ow in range(OW):
                win = xs[:, :, oh * strides[0]:oh * strides[0] + KH, ow * strides[1]:ow * strides[1] + KW]
                y[:, g * OCg:(g + 1) * OCg, oh, ow] = np.tensordot(win, ws, axes=([1, 2, 3], [1, 2, 3]))
    return y


CONV_CASES = [
    # N, C, H, W, OC, KH, KW, strides, pads, group
    (2, 4, 7, 6, 6, 3, 3, (1, 1), (1, 1), 1),
    (1, 6, 9, 8, 4, 3, 2, (2, 1), (0, 1), 2),
    (2, 8, 5, 5, 8, 3, 3, (1, 1), (1, 1), 8),     # depthwise
    (1, 3, 11, 11, 5, 7, 7, (2, 2), (3, 3), 1),   # stem-like
    (1, 5, 6, 7, 3, 1, 1, (2, 2), (0, 0), 1),     # strided pointwise
    (1, 2, 5, 4, 2, 3, 3, (2, 2), (0, 0, 1, 1), 1),  # asymmetric (what SAME_UPPER produces)
]


@pytest.mark.parametrize("case", CONV_CASES)
@pytest.mark.parametrize("wdt", [np.int8, np.uint8])
def test_conv_integer_vs_int64(oracle, case, wdt):
    N, C, H, W, OC, KH, KW, strides, pads, group = case
    rng = np.random.default_rng(3)
    x = rng.integers(0, 256, size=(N, C, H, W)).astype(np.uint8)
    lo, hi = (0, 256) if wdt == np.uint8 else (-128, 128)
    w = rng.integers(lo, hi, size=(OC, C // group, KH, KW)).astype(wdt)
    wz = rng.integers(lo, hi, size=OC).astype(wdt)
    xz = 131
    pads4 = pads if len(pads) == 4 else (pads[0], pads[1], pads[0], pads[1])
    want = np_conv_int64(x.astype(np.int64) - xz, w.astype(np.int64) - wz.astype(np.int64)[:, None, None, None],
                         strides, pads4, group)
    got = oracle.conv_integer(x, w, xz, wz, strides=strides, pads=pads, group=group)
    np.testing.assert_array_equal(got, want)
    # scalar w zero point and none
    want0 = np_conv_int64(x.astype(np.int64), w.astype(np.int64) - int(wz[0]), strides, pads4, group)
    np.testing.assert_array_equal(oracle.conv_integer(x, w, None, wz[:1], strides=strides, pads=pads, group=group), want0)


def test_same_upper_autopad(oracle):
    # CalculateAutoPad (runtime/chainerx_util.cc:276-311): out = ceil(in/stride); extra pad goes to the END
    assert oracle.same_upper_pads(5, 2, 3) == (1, 1)
    assert oracle.same_upper_pads(4, 2, 3) == (0, 1)
    assert oracle.same_upper_pads(28, 1, 3) == (1, 1)
    assert oracle.same_upper_pads(224, 2, 7) == (2, 3)
    rng = np.random.default_rng(4)
    x = rng.integers(0, 256, size=(1, 2, 4, 4)).astype(np.uint8)
    w = rng.integers(-128, 128, size=(3, 2, 3, 3)).astype(np.int8)
    got = oracle.conv_integer(x, w, 3, None, strides=(2, 2), pads=(0, 0), auto_pad="SAME_UPPER")
    want = np_conv_int64(x.astype(np.int64) - 3, w.astype(np.int64), (2, 2), (0, 0, 1, 1), 1)
    assert got.shape == (1, 3, 2, 2)
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("case", CONV_CASES)
@pytest.mark.parametrize("bias_mode", ["none", "reference_float", "onnx_int32"])
def test_qlinear_conv_int_equals_literal_on_power_of_two_scales(oracle, case, bias_mode):
    """With power-of-two scales and |acc| < 2^24 every fp32 product and partial sum
    of the literal path is exact, so both oracles must agree bit for bit."""
    N, C, H, W, OC, KH, KW, strides, pads, group = case
    rng = np.random.default_rng(5)
    x = rng.integers(0, 256, size=(N, C, H, W)).astype(np.uint8)
    w = rng.integers(-127, 128, size=(OC, C // group, KH, KW)).astype(np.int8)
    ws = (2.0 ** rng.integers(-9, -5, size=OC)).astype(np.float32)
    wz = np.zeros(OC, np.int8)
    bias = rng.integers(-1000, 1001, size=OC).astype(np.int32)
    kw = dict(strides=strides, pads=pads, group=group)
    if bias_mode == "none":
        kw.update(bias=None)
    elif bias_mode == "reference_float":
        kw.update(bias=bias, bias_mode=oracle.BIAS_REFERENCE_FLOAT)
    else:
        kw.update(bias=bias, bias_mode=oracle.BIAS_ONNX_INT32)
    args = (x, 2.0 ** -6, 128, w, ws, wz, 2.0 ** -3, 128)
    a = oracle.qlinear_conv_int(*args, **kw)
    b = oracle.qlinear_conv_literal(*args, **kw)
    np.testing.assert_array_equal(a, b)
    assert a.min() < a.max()  # not saturated into a constant


def test_qlinear_conv_int_closed_form_1x1(oracle):
    """1x1 conv, one channel: y = Q((x - xz) * (w - wz) * xs * ws) element by element."""
    x = np.arange(256, dtype=np.uint8).reshape(1, 1, 16, 16)
    w = np.array([[[[-3]]]], np.int8)
    xs, ws, ys, xz, yz = np.float32(0.02), np.float32(0.007), np.float32(0.05), 128, 128
    acc = (x.astype(np.int64) - xz) * -3
    v = acc.astype(np.float32) * np.float32(xs * ws)
    want = np_quantize(v, ys, yz, 0, 255)
    got = oracle.qlinear_conv_int(x, xs, xz, w, np.array([ws]), np.array([0], np.int8), ys, yz)
    np.testing.assert_array_equal(got.astype(np.int64), want)


def test_qlinear_matmul_relu_and_bias(oracle):
    rng = np.random.default_rng(6)
    a = rng.integers(0, 256, size=(32, 100)).astype(np.uint8)
    b = rng.integers(-127, 128, size=(100, 10)).astype(np.int8)
    bias = rng.integers(-500, 500, size=10).astype(np.int32)
    s_a, s_b, s_y = np.float32(1 / 255), np.float32(0.004), np.float32(0.02)
    acc = (a.astype(np.int64) - 128) @ b.astype(np.int64) + bias
    v = acc.astype(np.float32) * np.float32(s_a * s_b)
    want = np_quantize(v, s_y, 128, 0, 255)
    got = oracle.qlinear_matmul_int(a, s_a, 128, b, s_b, 0, s_y, 128, bias=bias)
    np.testing.assert_array_equal(got.astype(np.int64), want)
    got_relu = oracle.qlinear_matmul_int(a, s_a, 128, b, s_b, 0, s_y, 128, bias=bias, relu=True)
    np.testing.assert_array_equal(got_relu.astype(np.int64), np.maximum(want, 128))
    # fused Relu == Q(Relu(DQ(q))) spelled out with the element-wise oracle
    dq = oracle.dequantize_linear(got, s_y, 128)
    np.testing.assert_array_equal(oracle.quantize_linear(oracle.relu(dq), s_y, 128), got_relu)


def ulp_diff(a, b):
    a = np.asarray(a, np.float32).view(np.int32).astype(np.int64)
    b = np.asarray(b, np.float32).view(np.int32).astype(np.int64)
    a = np.where(a < 0, -(a & 0x7FFFFFFF), a)
    b = np.where(b < 0, -(b & 0x7FFFFFFF), b)
    return np.abs(a - b)


def test_elementwise_ops_against_float64(oracle):
    rng = np.random.default_rng(7)
    x = np.concatenate([rng.standard_normal(100000).astype(np.float32) * 3,
                        np.array([0, 1e-8, -1e-8, 0.5, 1, 21.9, 22, 30, -30, 88, -88, -104], np.float32)])
    x64 = x.astype(np.float64)
    assert ulp_diff(oracle.tanh(x), np.tanh(x64).astype(np.float32)).max() <= 2
    assert ulp_diff(oracle.exp(x), np.exp(x64).astype(np.float32)).max() <= 1
    assert ulp_diff(oracle.sigmoid(x), (1 / (1 + np.exp(-x64))).astype(np.float32)).max() <= 2
    np.testing.assert_array_equal(oracle.relu(x), np.maximum(x, 0))
    np.testing.assert_array_equal(oracle.clip(x, 0, 6), np.clip(x, 0, 6))
    a = rng.standard_normal(1024).astype(np.float32)
    x2 = rng.standard_normal((3, 5, 1024)).astype(np.float32)
    np.testing.assert_array_equal(oracle.binary(oracle.MUL, x2, a), x2 * a)
    np.testing.assert_array_equal(oracle.binary(oracle.ADD, x2, np.float32(2.5)), x2 + np.float32(2.5))
    np.testing.assert_array_equal(oracle.binary(oracle.SUB, a, x2), a - x2)
    col = rng.standard_normal((3, 5, 1)).astype(np.float32)   # not a trailing-axis broadcast: materialised
    np.testing.assert_array_equal(oracle.binary(oracle.DIV, x2, col), x2 / col)
    np.testing.assert_array_equal(oracle.round_half_even(np.array([0.5, 1.5, 2.5, -0.5, -1.5], np.float32)),
                                  np.array([0, 2, 2, -0, -2], np.float32))


def test_chain_matches_stepwise_numpy(oracle):
    rng = np.random.default_rng(8)
    x = rng.standard_normal((4, 8, 64)).astype(np.float32)
    c = rng.standard_normal((4, 8, 64)).astype(np.float32)
    a = rng.standard_normal(64).astype(np.float32)
    b = rng.standard_normal(64).astype(np.float32)
    prog = [("t0", "Mul", "x", "a"), ("t1", "Add", "t0", "b"), ("t2", "Tanh", "t1"), ("t3", "Sigmoid", "c"),
            ("t4", "Mul", "t2", "t3"), ("t5", "Add", "t4", "x"), ("y", "Relu", "t5")]
    env = oracle.run_chain(prog, dict(x=x, a=a, b=b, c=c))
    t1 = x * a + b  # numpy rounds after each op as well
    np.testing.assert_array_equal(env["t1"], t1)
    want = np.maximum(oracle.tanh(t1) * oracle.sigmoid(c) + x, 0)
    np.testing.assert_array_equal(env["y"], want)


def test_max_pool_window_in_the_padding_gives_what_quantizing_the_lowest_float_gives(oracle):
    """cover_all with pads can add a window that lies in the padding altogether.  Spelled out in
    float (ChainerX pads max-pooling with the lowest value): DequantizeLinear, maximum over a window
    padded with -inf, QuantizeLinear -> the clamp's lower end plus 0.5, truncated: 0 for uint8, -127 for int8."""
    rng = np.random.default_rng(17)
    for dt, lowest in ((np.uint8, 0), (np.int8, -127)):
        x = rng.integers(30, 100, size=(1, 2, 11, 16)).astype(dt)
        if dt == np.int8:
            x[0, 0, ::2] -= 110                               # negative codes as well
        got = oracle.max_pool_q8(x, (2, 3), (2, 2), (1, 1), True)
        assert got.shape == (1, 2, 7, 9)                      # rows start at -1, 1, ..., 11: the last one is past the image
        zp = 30 if dt == np.uint8 else -30
        dq = oracle.dequantize_linear(x, np.float32(0.05), zp)
        padded = np.full((1, 2, 11 + 1 + 3, 16 + 1 + 3), -np.inf, np.float32)
        padded[:, :, 1:12, 1:17] = dq
        want = np.empty((1, 2, 7, 9), np.float32)
        for oh in range(7):
            for ow in range(9):
                want[:, :, oh, ow] = padded[:, :, 2 * oh:2 * oh + 2, 2 * ow:2 * ow + 3].max(axis=(2, 3))
        assert np.isinf(want[:, :, 6, :]).all() and np.isfinite(want[:, :, :6, :]).all()
        assert (got[:, :, 6, :] == lowest).all()
        # the three float ops give the same bytes
        with np.errstate(all="ignore"):
            np.testing.assert_array_equal(got, oracle.quantize_linear(want, np.float32(0.05), zp, dt))


# --- pools between a DequantizeLinear and a QuantizeLinear (runtime/ops/pooling.cc:47-75) -------------
# Independent restatements: the oracle walks output pixels and gathers taps; these build an explicitly
# padded array and walk the taps, whole output planes at a time.

def np_dequantize(q, scale, zp):
    return (q.astype(np.float32) - np.float32(zp)) * np.float32(scale)


def np_average_pool_q8(x, x_scale, x_zp, kernel, strides, pads, y_scale, y_zp, y_dtype, count_include_pad, rne=False):
    N, C, H, W = x.shape
    (kh, kw), (sh, sw), (ph, pw) = kernel, strides, pads
    OH, OW = (H + 2 * ph - kh) // sh + 1, (W + 2 * pw - kw) // sw + 1
    val = np.zeros((N, C, H + 2 * ph, W + 2 * pw), np.float32)       # zero padding of the float tensor
    val[:, :, ph:ph + H, pw:pw + W] = np_dequantize(x, x_scale, x_zp)
    inside = np.zeros((H + 2 * ph, W + 2 * pw), np.int64)
    inside[ph:ph + H, pw:pw + W] = 1
    total = np.zeros((N, C, OH, OW), np.float32)
    count = np.zeros((OH, OW), np.int64)
    for i in range(kh):                                               # taps in (kh, kw) order, one fp32 addition each
        for j in range(kw):
            total = total + val[:, :, i:i + (OH - 1) * sh + 1:sh, j:j + (OW - 1) * sw + 1:sw]
            count += inside[i:i + (OH - 1) * sh + 1:sh, j:j + (OW - 1) * sw + 1:sw]
    if count_include_pad:
        count[:] = kh * kw
    mean = total / count.astype(np.float32)
    lo, hi = (0, 255) if y_dtype == np.uint8 else (-128, 127)
    if rne:
        s = mean / np.float32(y_scale)
        return np.clip(np.rint(s) + y_zp, lo, hi).astype(y_dtype)
    return np_quantize(mean, y_scale, y_zp, lo, hi).astype(y_dtype)


POOL_CASES = [  # kernel, strides, pads, H, W
    ((3, 3), (1, 1), (1, 1), 9, 11), ((2, 2), (2, 2), (0, 0), 8, 10), ((3, 2), (2, 1), (1, 0), 7, 9),
    ((5, 5), (3, 2), (2, 2), 13, 12), ((7, 7), (1, 1), (0, 0), 7, 7), ((1, 1), (1, 1), (0, 0), 4, 5),
    ((3, 3), (2, 2), (1, 1), 14, 14), ((2, 3), (1, 2), (1, 1), 5, 6)]


@pytest.mark.parametrize("x_dt,y_dt", [(np.uint8, np.uint8), (np.int8, np.int8), (np.uint8, np.int8), (np.int8, np.uint8)])
@pytest.mark.parametrize("include_pad", [False, True])
def test_average_pool_vs_numpy(oracle, x_dt, y_dt, include_pad):
    rng = np.random.default_rng(31)
    for kernel, strides, pads, H, W in POOL_CASES:
        lo, hi = (0, 256) if x_dt == np.uint8 else (-128, 128)
        x = rng.integers(lo, hi, size=(2, 3, H, W)).astype(x_dt)
        x_zp = int(rng.integers(lo, hi))
        y_zp = int(rng.integers(0, 256)) if y_dt == np.uint8 else int(rng.integers(-128, 128))
        x_scale, y_scale = np.float32(rng.uniform(0.01, 0.1)), np.float32(rng.uniform(0.01, 0.1))
        for rne in (False, True):
            got = oracle.average_pool_q8(x, x_scale, x_zp, kernel, strides, pads, y_scale, y_zp, y_dt, include_pad,
                                         oracle.ROUND_ONNX_RNE if rne else oracle.ROUND_REFERENCE)
            want = np_average_pool_q8(x, x_scale, x_zp, kernel, strides, pads, y_scale, y_zp, y_dt, include_pad, rne)
            np.testing.assert_array_equal(got, want, err_msg=str((kernel, strides, pads, rne)))


def test_average_pool_exact_family(oracle):
    """Power-of-two scales and small windows: every partial sum of the window is a small integer times
    the scale, exact in fp32 in any order, so the mean is fixed by integer arithmetic alone."""
    rng = np.random.default_rng(32)
    for kernel, strides, pads, H, W in POOL_CASES:
        for x_dt in (np.uint8, np.int8):
            lo, hi = (0, 256) if x_dt == np.uint8 else (-128, 128)
            x = rng.integers(lo, hi, size=(1, 2, H, W)).astype(x_dt)
            x_zp = int(rng.integers(lo, hi))
            for include_pad in (False, True):
                got = oracle.average_pool_q8(x, 0.125, x_zp, kernel, strides, pads, 0.25, 3, np.uint8, include_pad)
                OH, OW = got.shape[2:]
                want = np.empty_like(got)
                for c in range(2):
                    for oh in range(OH):
                        for ow in range(OW):
                            r0, c0 = oh * strides[0] - pads[0], ow * strides[1] - pads[1]
                            rows = range(max(r0, 0), min(r0 + kernel[0], H))
                            cols = range(max(c0, 0), min(c0 + kernel[1], W))
                            isum = sum(int(x[0, c, r, q]) - x_zp for r in rows for q in cols)   # exact integer
                            n = kernel[0] * kernel[1] if include_pad else len(rows) * len(cols)
                            mean = np.float32(isum * 0.125) / np.float32(n)                      # one rounding: the division
                            want[0, c, oh, ow] = np_quantize(np.array([mean], np.float32), 0.25, 3, 0, 255)[0]
                np.testing.assert_array_equal(got, want)


def test_average_pool_of_a_constant_image_is_the_constant(oracle):
    """x == c everywhere, window inside the image, one power-of-two scale on both sides: the sum of n equal
    values v is n*v exactly, the mean is v, and Q(DQ(c)) == c."""
    for c in (0, 1, 77, 128, 254, 255):
        x = np.full((1, 2, 8, 8), c, np.uint8)
        for kernel in ((2, 2), (3, 3), (8, 8), (5, 7)):
            got = oracle.average_pool_q8(x, 0.0625, 128, kernel, (1, 1), (0, 0), 0.0625, 128, np.uint8)
            assert (got == c).all()
    # with zero padding counted in, a corner window of a 3x3/pad 1 pool sees 4 of 9 taps
    x = np.full((1, 1, 6, 6), 200, np.uint8)
    got = oracle.average_pool_q8(x, 0.5, 128, (3, 3), (1, 1), (1, 1), 0.5, 128, np.uint8, True)
    corner = np_quantize(np.array([np.float32(4 * 36.0) / np.float32(9)], np.float32), 0.5, 128, 0, 255)[0]
    assert got[0, 0, 0, 0] == corner and got[0, 0, 2, 2] == 200
    got = oracle.average_pool_q8(x, 0.5, 128, (3, 3), (1, 1), (1, 1), 0.5, 128, np.uint8, False)
    assert (got == 200).all()


def test_global_average_pool_is_a_sequential_row_major_sum(oracle):
    """kernel = whole image: the (kh, kw) order is the image's row-major order, so the sum is the last
    entry of a float32 running sum (np.cumsum accumulates sequentially in the array's type)."""
    rng = np.random.default_rng(33)
    for H, W in ((7, 7), (4, 9), (14, 14)):
        x = rng.integers(0, 256, size=(3, 5, H, W)).astype(np.uint8)
        x_scale, y_scale = np.float32(0.0371), np.float32(0.0193)
        got = oracle.average_pool_q8(x, x_scale, 11, (H, W), (1, 1), (0, 0), y_scale, 4, np.uint8)
        run = np.cumsum(np_dequantize(x, x_scale, 11).reshape(3, 5, H * W), axis=2, dtype=np.float32)[:, :, -1]
        mean = run / np.float32(H * W)
        np.testing.assert_array_equal(got.reshape(3, 5), np_quantize(mean, y_scale, 4, 0, 255).astype(np.uint8))
        # the order matters for this input (otherwise the test above would pin nothing about it)
    x = rng.integers(0, 256, size=(64, 64, 7, 7)).astype(np.uint8)
    fwd = np.cumsum(np_dequantize(x, 0.0371, 11).reshape(64, 64, 49), axis=2, dtype=np.float32)[:, :, -1]
    rev = np.cumsum(np_dequantize(x, 0.0371, 11).reshape(64, 64, 49)[:, :, ::-1], axis=2, dtype=np.float32)[:, :, -1]
    assert (fwd != rev).any()


def np_max_pool_q8(x, kernel, strides, pads, cover_all):
    N, C, H, W = x.shape
    (kh, kw), (sh, sw), (ph, pw) = kernel, strides, pads
    if cover_all:
        OH, OW = -((H + 2 * ph - kh) // -sh) + 1, -((W + 2 * pw - kw) // -sw) + 1
    else:
        OH, OW = (H + 2 * ph - kh) // sh + 1, (W + 2 * pw - kw) // sw + 1
    lowest = np.iinfo(x.dtype).min
    # room for the windows that cover_all adds past the symmetric padding
    PH, PW = (OH - 1) * sh + kh, (OW - 1) * sw + kw
    pad = np.full((N, C, max(PH, H + 2 * ph), max(PW, W + 2 * pw)), lowest, np.int64)
    pad[:, :, ph:ph + H, pw:pw + W] = x
    out = np.full((N, C, OH, OW), lowest, np.int64)
    for i in range(kh):
        for j in range(kw):
            out = np.maximum(out, pad[:, :, i:i + (OH - 1) * sh + 1:sh, j:j + (OW - 1) * sw + 1:sw])
    if x.dtype == np.int8:
        out = out + (out < 0)   # the QuantizeLinear behind the pool: q + 0.5 truncates toward zero
    return out.astype(x.dtype)


def test_quantize_of_dequantize_is_the_code_for_uint8_and_one_more_for_negative_int8_codes():
    """Q(DQ(q)) over every code, a spread of scales and every zero point: q for uint8; q + (q < 0) for int8, where
    q + 0.5 is truncated toward zero by the cast (quantize.cc:16-35)."""
    rng = np.random.default_rng(36)
    scales = np.concatenate([rng.uniform(1e-4, 10.0, 40), 2.0 ** np.arange(-8, 4)]).astype(np.float32)
    for dt, lo, hi in ((np.uint8, 0, 255), (np.int8, -128, 127)):
        q = np.arange(lo, hi + 1).astype(dt)
        want = q.astype(np.int64) + ((q.astype(np.int64) < 0) if dt == np.int8 else 0)
        for scale in scales:
            for zp in range(lo, hi + 1, 5):
                np.testing.assert_array_equal(np_quantize(np_dequantize(q, scale, zp), scale, zp, lo, hi), want, err_msg=str((dt, scale, zp)))


@pytest.mark.parametrize("dt", [np.uint8, np.int8])
@pytest.mark.parametrize("cover_all", [False, True])
def test_max_pool_vs_numpy(oracle, dt, cover_all):
    rng = np.random.default_rng(34)
    info = np.iinfo(dt)
    for kernel, strides, pads, H, W in POOL_CASES + [((3, 3), (2, 2), (0, 0), 112, 112)]:
        x = rng.integers(info.min, info.max + 1, size=(2, 3, H, W)).astype(dt)
        got = oracle.max_pool_q8(x, kernel, strides, pads, cover_all)
        np.testing.assert_array_equal(got, np_max_pool_q8(x, kernel, strides, pads, cover_all), err_msg=str((kernel, strides, pads)))
    # kernel = whole image: the maximum of each plane
    x = rng.integers(info.min, info.max + 1, size=(2, 3, 6, 5)).astype(dt)
    m = x.max(axis=(2, 3)).astype(np.int64)
    np.testing.assert_array_equal(oracle.max_pool_q8(x, (6, 5), (1, 1), (0, 0), cover_all).reshape(2, 3), m + ((m < 0) if dt == np.int8 else 0))


@pytest.mark.parametrize("dt", [np.uint8, np.int8])
def test_max_pool_on_codes_equals_the_three_float_ops(oracle, dt):
    """DequantizeLinear -> MaxPool over a -inf padded float tensor -> QuantizeLinear, spelled out, for any zero point
    and window: the maximum of the codes for uint8 (increasing dequantization, Q(DQ(q)) == q), one more for a negative
    maximum for int8."""
    rng = np.random.default_rng(35)
    info = np.iinfo(dt)
    for kernel, strides, pads, H, W in POOL_CASES:
        x = rng.integers(info.min, info.max + 1, size=(1, 2, H, W)).astype(dt)
        zp = int(rng.integers(info.min, info.max + 1))
        scale = np.float32(rng.uniform(0.01, 0.2))
        got = oracle.max_pool_q8(x, kernel, strides, pads, False)
        OH, OW = got.shape[2:]
        val = np.full((1, 2, H + 2 * pads[0], W + 2 * pads[1]), -np.inf, np.float32)
        val[:, :, pads[0]:pads[0] + H, pads[1]:pads[1] + W] = np_dequantize(x, scale, zp)
        want = np.full((1, 2, OH, OW), -np.inf, np.float32)
        for i in range(kernel[0]):
            for j in range(kernel[1]):
                want = np.maximum(want, val[:, :, i:i + (OH - 1) * strides[0] + 1:strides[0], j:j + (OW - 1) * strides[1] + 1:strides[1]])
        with np.errstate(all="ignore"):
            np.testing.assert_array_equal(got, np_quantize(want, scale, zp, info.min, info.max).astype(dt))


# --- Gemm / Linear / Flatten (runtime/ops/math.cc:160-177, connection.cc:12-15, manipulation.cc:20-28) ---
# What numpy fixes: the value up to the rounding of a float32 sum (float64 product, bound from the row
# norms), every bit on integer-valued operands (each partial sum is exact, so no order can differ), the
# alpha / beta / c branches, and the order on one row (a sequential float32 running sum).

def test_gemm_against_float64_within_the_float32_sum_bound(oracle):
    rng = np.random.default_rng(51)
    for M, N, K, ta, tb in ((5, 7, 33, False, False), (16, 3, 100, True, False), (3, 9, 64, False, True), (8, 8, 17, True, True)):
        a = rng.standard_normal((K, M) if ta else (M, K)).astype(np.float32)
        b = rng.standard_normal((N, K) if tb else (K, N)).astype(np.float32)
        got = oracle.gemm(a, b, trans_a=ta, trans_b=tb)
        A = (a.T if ta else a).astype(np.float64)
        B = (b.T if tb else b).astype(np.float64)
        exact = A @ B
        bound = (K + 1) * 2.0 ** -24 * (np.abs(A) @ np.abs(B))   # a float32 sum of K products
        assert got.dtype == np.float32 and got.shape == (M, N)
        assert (np.abs(got - exact) <= bound + 1e-30).all()
        # a transposed operand is the product of the transposed matrix, bit for bit
        np.testing.assert_array_equal(got, oracle.gemm(np.ascontiguousarray(A.astype(np.float32)), np.ascontiguousarray(B.astype(np.float32))))


def test_gemm_is_exact_on_integer_valued_operands(oracle):
    """Every product and partial sum is an integer below 2^24: float32 holds them exactly, so any order of
    summation gives numpy's int64 result, and a dropped term or a wrong index does not."""
    rng = np.random.default_rng(52)
    a = rng.integers(-30, 31, size=(9, 40)).astype(np.float32)
    b = rng.integers(-30, 31, size=(40, 11)).astype(np.float32)
    c = rng.integers(-100, 101, size=(11,)).astype(np.float32)
    want = a.astype(np.int64) @ b.astype(np.int64)
    np.testing.assert_array_equal(oracle.gemm(a, b), want.astype(np.float32))
    np.testing.assert_array_equal(oracle.gemm(a.T.copy(), b.T.copy(), trans_a=True, trans_b=True), want.astype(np.float32))
    np.testing.assert_array_equal(oracle.gemm(a, b, c), (want + c.astype(np.int64)).astype(np.float32))
    np.testing.assert_array_equal(oracle.gemm(a, b, c, alpha=2.0, beta=3.0), (2 * want + 3 * c.astype(np.int64)).astype(np.float32))
    # c broadcasts as numpy does: a column, a full matrix, a single element
    col = rng.integers(-9, 10, size=(9, 1)).astype(np.float32)
    full = rng.integers(-9, 10, size=(9, 11)).astype(np.float32)
    np.testing.assert_array_equal(oracle.gemm(a, b, col), (want + col.astype(np.int64)).astype(np.float32))
    np.testing.assert_array_equal(oracle.gemm(a, b, full), (want + full.astype(np.int64)).astype(np.float32))
    np.testing.assert_array_equal(oracle.gemm(a, b, np.float32([[5]])), (want + 5).astype(np.float32))
    # beta == 0 leaves c out altogether, even a c of NaNs
    np.testing.assert_array_equal(oracle.gemm(a, b, np.full(11, np.nan, np.float32), beta=0.0), want.astype(np.float32))
    # Linear = x . w^T + b over the flattened batch axes
    x = rng.integers(-5, 6, size=(2, 3, 4, 5)).astype(np.float32)
    w = rng.integers(-5, 6, size=(6, 20)).astype(np.float32)
    bias = rng.integers(-5, 6, size=(6,)).astype(np.float32)
    np.testing.assert_array_equal(oracle.linear(x, w, bias, n_batch_axes=2),
                                  (x.reshape(6, 20).astype(np.int64) @ w.T.astype(np.int64) + bias.astype(np.int64)).reshape(2, 3, 6).astype(np.float32))
    np.testing.assert_array_equal(oracle.linear(x.reshape(2, 60), rng.integers(-2, 3, size=(4, 60)).astype(np.float32) * 0 + 1),
                                  np.repeat(x.reshape(2, 60).sum(axis=1, keepdims=True), 4, axis=1))


def test_gemm_rounds_once_per_operation_in_the_order_of_math_cc(oracle):
    """r = Dot; r *= alpha; xc = c * beta; r + xc: each step rounds to float32 on its own (no fused
    multiply-add), and the dot product of a row is the sequential float32 running sum."""
    rng = np.random.default_rng(53)
    a = rng.standard_normal((4, 300)).astype(np.float32)
    b = rng.standard_normal((300, 5)).astype(np.float32)
    c = rng.standard_normal((5,)).astype(np.float32)
    alpha, beta = np.float32(0.7), np.float32(-1.3)
    prods = a[:, :, None] * b[None, :, :]                       # float32 products
    dot = np.zeros((4, 5), np.float32)
    for k in range(300):
        dot = dot + prods[:, k, :]                              # one float32 addition each, ascending k
    np.testing.assert_array_equal(oracle.gemm(a, b), dot)
    np.testing.assert_array_equal(oracle.gemm(a, b, c, alpha=alpha, beta=beta), dot * alpha + c * beta)
    np.testing.assert_array_equal(oracle.gemm(a, b, c, alpha=alpha), dot * alpha + c)
    np.testing.assert_array_equal(oracle.gemm(a, b, c, beta=beta), dot + c * beta)
    # the order matters on this data: the same terms added in descending k give other bits somewhere
    back = np.zeros((4, 5), np.float32)
    for k in reversed(range(300)):
        back = back + prods[:, k, :]
    assert (back != dot).any()


def test_flatten(oracle):
    x = np.arange(2 * 3 * 4 * 5).reshape(2, 3, 4, 5).astype(np.float32)
    for axis, shape in ((0, (1, 120)), (1, (2, 60)), (2, (6, 20)), (3, (24, 5)), (-1, (24, 5)), (-3, (2, 60))):
        got = oracle.flatten(x, axis)
        assert got.shape == shape
        np.testing.assert_array_equal(got.ravel(), x.ravel())
    # a channels-last view flattens in its logical (NCHW) order
    nhwc = np.ascontiguousarray(x.transpose(0, 2, 3, 1)).transpose(0, 3, 1, 2)
    np.testing.assert_array_equal(oracle.flatten(nhwc, 1), x.reshape(2, 60))


# --- float pools (runtime/ops/pooling.cc:47-75) ---

def np_max_pool_f32(x, kernel, strides, pads, cover_all):
    N, C, H, W = x.shape
    (kh, kw), (sh, sw), (ph, pw) = kernel, strides, pads
    if cover_all:
        OH, OW = -((H + 2 * ph - kh) // -sh) + 1, -((W + 2 * pw - kw) // -sw) + 1
    else:
        OH, OW = (H + 2 * ph - kh) // sh + 1, (W + 2 * pw - kw) // sw + 1
    lowest = np.finfo(np.float32).min
    PH, PW = (OH - 1) * sh + kh, (OW - 1) * sw + kw
    pad = np.full((N, C, max(PH, H + 2 * ph), max(PW, W + 2 * pw)), lowest, np.float32)
    pad[:, :, ph:ph + H, pw:pw + W] = x
    out = np.full((N, C, OH, OW), lowest, np.float32)
    for i in range(kh):
        for j in range(kw):
            out = np.maximum(out, pad[:, :, i:i + (OH - 1) * sh + 1:sh, j:j + (OW - 1) * sw + 1:sw])
    return out


@pytest.mark.parametrize("cover_all", [False, True])
def test_float_max_pool_vs_numpy(oracle, cover_all):
    rng = np.random.default_rng(61)
    for kernel, strides, pads, H, W in POOL_CASES:
        x = rng.standard_normal((2, 3, H, W)).astype(np.float32)
        np.testing.assert_array_equal(oracle.max_pool(x, kernel, strides, pads, cover_all), np_max_pool_f32(x, kernel, strides, pads, cover_all),
                                      err_msg=str((kernel, strides, pads)))
    x = rng.standard_normal((2, 3, 6, 5)).astype(np.float32)
    np.testing.assert_array_equal(oracle.max_pool(x, (6, 5), (1, 1), (0, 0), cover_all).reshape(2, 3), x.max(axis=(2, 3)))


@pytest.mark.parametrize("include_pad", [False, True])
def test_float_average_pool_vs_numpy(oracle, include_pad):
    rng = np.random.default_rng(62)
    for kernel, strides, pads, H, W in POOL_CASES:
        x = rng.standard_normal((2, 3, H, W)).astype(np.float32)
        (kh, kw), (sh, sw), (ph, pw) = kernel, strides, pads
        OH, OW = (H + 2 * ph - kh) // sh + 1, (W + 2 * pw - kw) // sw + 1
        val = np.zeros((2, 3, H + 2 * ph, W + 2 * pw), np.float32)
        val[:, :, ph:ph + H, pw:pw + W] = x
        inside = np.zeros((H + 2 * ph, W + 2 * pw), np.int64)
        inside[ph:ph + H, pw:pw + W] = 1
        total = np.zeros((2, 3, OH, OW), np.float32)
        count = np.zeros((OH, OW), np.int64)
        for i in range(kh):                       # taps in (kh, kw) order, one float32 addition each; padding adds 0.0f
            for j in range(kw):
                total = total + val[:, :, i:i + (OH - 1) * sh + 1:sh, j:j + (OW - 1) * sw + 1:sw]
                count = count + inside[i:i + (OH - 1) * sh + 1:sh, j:j + (OW - 1) * sw + 1:sw]
        div = np.float32(kh * kw) if include_pad else count.astype(np.float32)
        np.testing.assert_array_equal(oracle.average_pool(x, kernel, strides, pads, include_pad), total / div, err_msg=str((kernel, strides, pads)))
    # integer-valued image: every sum is exact, so the mean is numpy's whatever the order
    xi = rng.integers(-50, 51, size=(1, 2, 9, 9)).astype(np.float32)
    got = oracle.average_pool(xi, (3, 3), (3, 3), (0, 0), include_pad)
    np.testing.assert_array_equal(got, (xi.reshape(1, 2, 3, 3, 3, 3).transpose(0, 1, 2, 4, 3, 5).reshape(1, 2, 3, 3, 9).sum(axis=-1) / np.float32(9)).astype(np.float32))
    # whole-image window: the sequential float32 running sum of the pixels in storage order
    xg = rng.standard_normal((1, 2, 7, 7)).astype(np.float32)
    seq = np.cumsum(xg.reshape(1, 2, 49), axis=-1, dtype=np.float32)[..., -1] / np.float32(49)
    np.testing.assert_array_equal(oracle.average_pool(xg, (7, 7), (1, 1), (0, 0), include_pad).reshape(1, 2), seq)


def test_fixed_batch_norm_pins(oracle):
    """orc_fixed_batch_norm_f32 against float64 (five float32 roundings: the bound below), bit for bit where every
    step is exact, against the same steps in numpy float32, and the op's adjustment of a small epsilon
    (runtime/ops/normalization.cc:217-218)."""
    rng = np.random.default_rng(71)
    for shape in [(4, 6, 5, 7), (3, 5), (2, 4, 9)]:
        C = shape[1]
        x = (rng.standard_normal(shape) * 3).astype(np.float32)
        s, bias, mean = (rng.standard_normal(C).astype(np.float32) for _ in range(3))
        var = rng.uniform(0.01, 4.0, C).astype(np.float32)
        bc = (1, C) + (1,) * (len(shape) - 2)
        for eps in (1e-3, 1e-5, 0.0):
            eff = np.float32(eps) if eps > 1e-5 else np.float32(1e-5 + 1e-12)
            got = oracle.fixed_batch_norm(x, s, bias, mean, var, eps)
            # the same five operations in numpy float32
            inv = np.float32(1) / np.sqrt(var + eff)
            steps = ((x - mean.reshape(bc)) * inv.reshape(bc)) * s.reshape(bc) + bias.reshape(bc)
            np.testing.assert_array_equal(got, steps)
            f8 = np.float64
            scaled = (x.astype(f8) - mean.reshape(bc).astype(f8)) / np.sqrt(var.reshape(bc).astype(f8) + f8(eff)) * s.reshape(bc).astype(f8)
            exact = scaled + bias.reshape(bc).astype(f8)
            bound = 2.0 ** -24 * (5 * np.abs(scaled) + np.abs(exact)) + 1e-37
            assert (np.abs(got - exact) <= bound).all()
    # exact family: integer deviations, var + eps a power of four, power-of-two scales, integer biases
    x = rng.integers(-100, 101, size=(2, 4, 3, 3)).astype(np.float32)
    mean = np.array([3, -7, 0, 12], np.float32)
    var = np.array([0.0, 0.75, 3.75, 15.75], np.float32)       # + 0.25 = 0.25, 1, 4, 16
    s = np.array([2.0, -0.5, 4.0, 1.0], np.float32)
    bias = np.array([5, -3, 0, 100], np.float32)
    want = (x - mean.reshape(1, 4, 1, 1)) * (s / np.array([0.5, 1, 2, 4], np.float32)).reshape(1, 4, 1, 1) + bias.reshape(1, 4, 1, 1)
    np.testing.assert_array_equal(oracle.fixed_batch_norm(x, s, bias, mean, var, 0.25), want)
    # epsilon at or below 1e-5 is replaced: with var = 0 the replaced value shows
    z = np.zeros(4, np.float32)
    a = oracle.fixed_batch_norm(x, s, z, z, z, 1e-5)
    b = oracle.fixed_batch_norm(x, s, z, z, z, float(np.float32(1e-5 + 1e-12)) + 1e-9)   # just above: taken as it is
    c = oracle.fixed_batch_norm(x, s, z, z, z, 0.0)
    np.testing.assert_array_equal(a, c)
    assert np.float32(1e-5 + 1e-12) > np.float32(1e-5)
    naive = (x * (np.float32(1) / np.sqrt(np.float32(1e-5)))) * s.reshape(1, 4, 1, 1)
    assert not np.array_equal(a, naive)
    assert np.allclose(a, b, rtol=1e-3)


def test_float_conv_pins(oracle):
    """orc_conv_f32 against float64 (bound of a K-term float32 sum), bit for bit on integer-valued operands (every
    sum exact whatever its order) with groups, strides and pads, and against orc_gemm_f32 on the explicitly
    expanded matrix (the same k order)."""
    import torch
    rng = np.random.default_rng(81)
    cases = [  # N, C, H, W, OC, KH, KW, strides, pads, group
        (2, 3, 9, 8, 4, 3, 3, (1, 1), (1, 1), 1), (1, 4, 7, 7, 6, 1, 1, (2, 2), (0, 0), 2), (2, 6, 8, 8, 6, 3, 2, (2, 1), (0, 1), 6),
        (1, 8, 5, 5, 4, 5, 5, (1, 1), (2, 2), 4), (3, 2, 6, 6, 5, 2, 2, (2, 2), (0, 0), 1)]
    for N, C, H, W, OC, KH, KW, strides, pads, group in cases:
        x = rng.standard_normal((N, C, H, W)).astype(np.float32)
        w = rng.standard_normal((OC, C // group, KH, KW)).astype(np.float32)
        b = rng.standard_normal(OC).astype(np.float32)
        got = oracle.conv(x, w, b, strides, pads, group)
        tx = torch.from_numpy
        exact = torch.nn.functional.conv2d(tx(x).double(), tx(w).double(), tx(b).double(), strides, pads, 1, group).numpy()
        mag = torch.nn.functional.conv2d(tx(np.abs(x)).double(), tx(np.abs(w)).double(), None, strides, pads, 1, group).numpy() + np.abs(b).reshape(1, -1, 1, 1)
        K = (C // group) * KH * KW
        assert got.shape == exact.shape and (np.abs(got - exact) <= (K + 2) * 2.0 ** -24 * mag + 1e-30).all()
        xi = rng.integers(-8, 9, size=x.shape).astype(np.float32)
        wi = rng.integers(-8, 9, size=w.shape).astype(np.float32)
        bi = rng.integers(-50, 51, size=OC).astype(np.float32)
        want = torch.nn.functional.conv2d(tx(xi).double(), tx(wi).double(), tx(bi).double(), strides, pads, 1, group).numpy()
        np.testing.assert_array_equal(oracle.conv(xi, wi, bi, strides, pads, group), want.astype(np.float32))
        np.testing.assert_array_equal(oracle.conv(xi, wi, None, strides, pads, group), (want - bi.reshape(1, -1, 1, 1)).astype(np.float32))
    # the same order as a matrix product over the expanded matrix with k = (c, kh, kw)
    x = rng.standard_normal((2, 3, 6, 6)).astype(np.float32)
    w = rng.standard_normal((5, 3, 3, 3)).astype(np.float32)
    xp = np.pad(x, ((0, 0), (0, 0), (1, 1), (1, 1)))
    col = np.stack([xp[:, :, i:i + 6, j:j + 6] for i in range(3) for j in range(3)], axis=2)      # [N, C, 9, OH, OW]
    col = col.transpose(0, 3, 4, 1, 2).reshape(2 * 36, 27)
    want = oracle.gemm(col, w.reshape(5, 27), trans_b=True).reshape(2, 6, 6, 5).transpose(0, 3, 1, 2)
    np.testing.assert_array_equal(oracle.conv(x, w, None, (1, 1), (1, 1)), want)


def test_softmax_pins(oracle):
    """orc_softmax_f32 against float64, rows summing to 1 within `len` roundings, shift invariance where the shift is
    exact, and the two axis semantics of RunSoftmax (runtime/ops/activation.cc:66-89) against each other."""
    rng = np.random.default_rng(91)
    for shape, axis in [((4, 10), 1), ((3, 5, 7), 1), ((3, 5, 7), 2), ((2, 3, 4, 5), 1), ((6,), 0), ((2, 1000), -1)]:
        x = (rng.standard_normal(shape) * 4).astype(np.float32)
        for onnx in (True, False):
            got = oracle.softmax(x, axis, onnx)
            ax = axis % x.ndim
            red = tuple(range(ax, x.ndim)) if onnx else (ax,)
            x8 = x.astype(np.float64)
            e = np.exp(x8 - x8.max(axis=red, keepdims=True))
            exact = e / e.sum(axis=red, keepdims=True)
            n = int(np.prod([x.shape[d] for d in red]))
            assert (np.abs(got - exact) <= (n + 8) * 2.0 ** -24 * exact + 1e-45).all()
            assert np.abs(got.astype(np.float64).sum(axis=red) - 1).max() <= (2 * n + 8) * 2.0 ** -24
            # integer-valued rows: adding 16 changes nothing in x - max, so nothing in the result
            xi = rng.integers(-20, 21, size=shape).astype(np.float32)
            np.testing.assert_array_equal(oracle.softmax(xi + np.float32(16), axis, onnx), oracle.softmax(xi, axis, onnx))
    x = (rng.standard_normal((3, 4, 5)) * 2).astype(np.float32)
    # ONNX semantics at axis 1 = the reduction over the last axis of the array reshaped to [3, 20]
    np.testing.assert_array_equal(oracle.softmax(x, 1, True), oracle.softmax(x.reshape(3, 20), 1, False).reshape(3, 4, 5))
    # chainer semantics at axis 1 = over the last axis of the transposed array
    np.testing.assert_array_equal(oracle.softmax(x, 1, False), oracle.softmax(x.transpose(0, 2, 1), 2, False).transpose(0, 2, 1))
    # one element: exactly 1; a NaN spreads over its row only
    assert oracle.softmax(np.array([[3.5]], np.float32), 1).tolist() == [[1.0]]
    xn = np.array([[1, np.nan, 2], [1, 2, 3]], np.float32)
    got = oracle.softmax(xn, 1)
    assert np.isnan(got[0]).all() and not np.isnan(got[1]).any()
