"""The int8 MFMA implicit-GEMM path of QLinearConv / ConvInteger / QLinearMatMul /
MatMulInteger, bit-exact against the integer-accumulating oracle, at shapes chosen to
cross every tiling edge: K tails (C not a multiple of 64), output channels and pixels
that do not fill a tile, strides, padding, 7x7 kernels, both operand layouts."""
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


def make_case(rng, N, C, H, W, OC, KH, KW, xdt=np.uint8):
    lo, hi = (0, 256) if xdt == np.uint8 else (-128, 128)
    x = rng.integers(lo, hi, size=(N, C, H, W)).astype(xdt)
    w = rng.integers(-127, 128, size=(OC, C, KH, KW)).astype(np.int8)
    ws = rng.uniform(0.001, 0.01, size=OC).astype(np.float32)
    bias = rng.integers(-1000, 1001, size=OC).astype(np.int32)
    ys = np.float32(0.02 * 0.0055 * 74 * 73 * np.sqrt(C * KH * KW) / 40)
    return x, w, ws, np.zeros(OC, np.int8), bias, ys


MFMA_CASES = [
    # N, C, H, W, OC, KH, KW, strides, pads
    (2, 128, 28, 28, 128, 3, 3, (1, 1), (1, 1)),     # the stage-3 ResNet block shape, reduced batch
    (1, 64, 56, 56, 64, 1, 1, (1, 1), (0, 0)),       # pointwise
    (2, 256, 14, 14, 512, 1, 1, (2, 2), (0, 0)),     # strided pointwise shortcut
    (1, 96, 9, 11, 40, 3, 3, (1, 1), (1, 1)),        # K tail (96 = 64 + 32), OC and pixels ragged
    (1, 16, 13, 13, 24, 3, 3, (2, 2), (1, 1)),       # one 16-byte chunk per tap
    (1, 3, 37, 37, 64, 7, 7, (2, 2), (3, 3)),        # stem-like: 3 channels (NCHW input only)
    (3, 64, 7, 7, 1000, 1, 1, (1, 1), (0, 0)),       # OC not a multiple of 16
    (1, 512, 7, 7, 512, 3, 3, (1, 1), (1, 1)),       # K = 4608, few pixels
]


@pytest.mark.parametrize("case", MFMA_CASES)
@pytest.mark.parametrize("layout", ["nchw", "channels_last"])
def test_qlinear_conv_mfma(g, oracle, case, layout):
    N, C, H, W, OC, KH, KW, strides, pads = case
    if layout == "channels_last" and C % 16:
        pytest.skip("channels-last views with a pitch below 16 bytes take the direct kernel (covered elsewhere)")
    rng = np.random.default_rng(31)
    x, w, ws, wz, bias, ys = make_case(rng, N, C, H, W, OC, KH, KW)
    want = oracle.qlinear_conv_int(x, 0.02, 128, w, ws, wz, ys, 128, np.uint8, bias=bias, strides=strides, pads=pads,
                                   bias_mode=oracle.BIAS_ONNX_INT32)
    assert want.min() < 64 and want.max() > 192          # the output range is really used
    xd = g.dev(x)
    if layout == "channels_last":
        xd = g.to_channels_last(xd)
    got = g.ops.QLinearConv(xd, 0.02, 128, g.dev(w), g.dev(ws), g.dev(wz), ys, 128, g.dev(bias), strides=strides,
                            pads=pads, flags=g.capi.BIAS_ONNX_INT32)
    np.testing.assert_array_equal(g.host(got), want)


@pytest.mark.parametrize("xdt", [np.uint8, np.int8])
def test_mfma_zero_points_bias_modes_and_plan_reuse(g, oracle, xdt):
    rng = np.random.default_rng(32)
    x, w, ws, wz, bias, ys = make_case(rng, 2, 64, 12, 12, 96, 3, 3, xdt)
    plan = g.ops.QLinearConvPlan(g.dev(w), g.dev(ws), g.dev(wz), g.dev(bias), pads=(1, 1))
    xd = g.to_channels_last(g.dev(x))
    for xz, yz, ydt, flags, okw in [
            (128 if xdt == np.uint8 else 0, 128, np.uint8, 0, dict(bias_mode=oracle.BIAS_REFERENCE_FLOAT)),
            (3, 0, np.uint8, g.capi.BIAS_ONNX_INT32 | g.capi.FUSE_RELU, dict(bias_mode=oracle.BIAS_ONNX_INT32)),
            (100, -5, np.int8, g.capi.BIAS_ONNX_INT32 | g.capi.ROUND_ONNX_RNE,
             dict(bias_mode=oracle.BIAS_ONNX_INT32, round_mode=oracle.ROUND_ONNX_RNE))]:
        want = oracle.qlinear_conv_int(x, 0.02, xz, w, ws, wz, ys, yz, ydt, bias=bias, pads=(1, 1), **okw)
        if flags & g.capi.FUSE_RELU:
            want = np.maximum(want, yz).astype(ydt)
        got = plan.run(xd, 0.02, xz, ys, yz, TDT[ydt], flags=flags)
        assert got.permute(0, 2, 3, 1).is_contiguous()
        np.testing.assert_array_equal(g.host(got), want)
    # the same plan on another input size, and no bias at all through the one-shot entry point
    x2 = rng.integers(0, 256, size=(1, 64, 5, 20)).astype(np.uint8) if xdt == np.uint8 else \
        rng.integers(-128, 128, size=(1, 64, 5, 20)).astype(np.int8)
    want = oracle.qlinear_conv_int(x2, 0.02, 7, w, ws, wz, ys, 128, np.uint8, bias=bias, pads=(1, 1),
                                   bias_mode=oracle.BIAS_ONNX_INT32)
    np.testing.assert_array_equal(g.host(plan.run(g.dev(x2), 0.02, 7, ys, 128, flags=g.capi.BIAS_ONNX_INT32)), want)
    plan.close()
    want = oracle.qlinear_conv_int(x, 0.02, 7, w, ws[:1], wz[:1], ys, 128, np.uint8, pads=(1, 1))
    got = g.ops.QLinearConv(xd, 0.02, 7, g.dev(w), g.dev(ws[:1].reshape(())), g.dev(wz[:1].reshape(())), ys, 128, pads=(1, 1))
    np.testing.assert_array_equal(g.host(got), want)


def test_conv_integer_mfma(g, oracle):
    rng = np.random.default_rng(33)
    x, w, _, _, _, _ = make_case(rng, 2, 80, 10, 9, 72, 3, 3)
    want = oracle.conv_integer(x, w, 131, None, strides=(1, 1), pads=(1, 1))
    got = g.ops.ConvInteger(g.to_channels_last(g.dev(x)), g.dev(w), 131, None, pads=(1, 1))
    np.testing.assert_array_equal(g.host(got), want)
    got = g.ops.ConvInteger(g.dev(x), g.dev(w), 131, g.dev(np.zeros(72, np.int8)), pads=(1, 1),
                            out=torch.empty((2, 10, 9, 72), dtype=torch.int32, device="cuda").permute(0, 3, 1, 2))
    np.testing.assert_array_equal(g.host(got), want)


@pytest.mark.parametrize("M,K,N", [(256, 784, 100), (1000, 2048, 1000), (77, 64, 10), (4096, 128, 512)])
def test_matmul_mfma(g, oracle, M, K, N):
    rng = np.random.default_rng(34)
    a = rng.integers(0, 256, size=(M, K)).astype(np.uint8)
    b = rng.integers(-127, 128, size=(K, N)).astype(np.int8)
    bias = rng.integers(-3000, 3000, size=N).astype(np.int32)
    ys = np.float32(0.004 * 0.01 * 74 * 73 * np.sqrt(K) / 40)
    want = oracle.qlinear_matmul_int(a, 0.004, 128, b, 0.01, 0, ys, 128, bias=bias, relu=True)
    got = g.ops.QLinearMatMul(g.dev(a), 0.004, 128, g.dev(b), 0.01, 0, ys, 128, g.dev(bias), flags=g.capi.FUSE_RELU)
    np.testing.assert_array_equal(g.host(got), want)
    assert want.max() > 192
    want = oracle.matmul_integer(a, b, np.array([128], np.uint8), None)
    got = g.ops.MatMulInteger(g.dev(a), g.dev(b), g.dev(np.array([128], np.uint8)), None)
    np.testing.assert_array_equal(g.host(got), want)


def test_full_size_conv_properties(g, oracle):
    """x uint8 [32,128,28,28], w int8 [128,128,3,3], per-channel scales, int32 bias: the whole
    output against the oracle on four images, and for all 32 through properties of the integer
    contraction that do not depend on size (linearity in the weights, shift of the zero point)."""
    rng = np.random.default_rng(2)
    x = rng.integers(0, 256, size=(32, 128, 28, 28)).astype(np.uint8)
    w = rng.integers(-127, 128, size=(128, 128, 3, 3)).astype(np.int8)
    ws = rng.uniform(0.001, 0.01, size=128).astype(np.float32)
    wz = np.zeros(128, np.int8)
    bias = rng.integers(-1000, 1001, size=128).astype(np.int32)
    xd = g.to_channels_last(g.dev(x))
    got = g.ops.QLinearConv(xd, 0.02, 128, g.dev(w), g.dev(ws), g.dev(wz), 0.05, 128, g.dev(bias), pads=(1, 1),
                            flags=g.capi.BIAS_ONNX_INT32)
    sel = [0, 13, 14, 31]
    want = oracle.qlinear_conv_int(x[sel], 0.02, 128, w, ws, wz, 0.05, 128, np.uint8, bias=bias, pads=(1, 1),
                                   bias_mode=oracle.BIAS_ONNX_INT32)
    np.testing.assert_array_equal(g.host(got)[sel], want)
    # integer contraction: conv(x, w1 + w2) == conv(x, w1) + conv(x, w2), and
    # conv(x; zp) - conv(x; zp') == (zp' - zp) * (sum of the taps inside the image)
    w1 = (w // 2).astype(np.int8)
    w2 = (w - w1).astype(np.int8)
    ci = lambda wt, zp: g.ops.ConvInteger(xd, g.dev(wt), zp, None, pads=(1, 1))
    full, p1, p2 = ci(w, 128), ci(w1, 128), ci(w2, 128)
    torch.cuda.synchronize()
    assert torch.equal(full, p1 + p2)
    ones = torch.ones_like(xd)
    taps = g.ops.ConvInteger(ones, g.dev(w), 0, None, pads=(1, 1))   # per-position sum of in-image taps
    assert torch.equal(ci(w, 100) - full, 28 * taps)


PADDED_WINDOWS = [
    # N, C, H, W, OC, KH, KW, strides, pads
    (2, 32, 1, 1, 32, 3, 3, (1, 1), (1, 1)),      # a window that leaves the image on all four sides
    (2, 64, 2, 5, 48, 3, 3, (1, 1), (1, 1)),      # ... above and below at once
    (1, 64, 8, 8, 64, 3, 3, (2, 2), (1, 1)),      # stride 2 over an even image: nothing below or to the right
    (1, 64, 9, 7, 64, 3, 3, (2, 2), (1, 1)),      # ... over an odd one
    (1, 256, 6, 6, 64, 1, 1, (1, 1), (1, 1)),     # a single tap that can lie outside altogether
    (1, 64, 6, 6, 32, 2, 2, (1, 1), (1, 1)),
    (1, 16, 10, 10, 32, 5, 5, (1, 1), (1, 1)),    # 25 taps, one row or column outside per side
    (1, 16, 10, 10, 32, 5, 5, (1, 1), (2, 2)),    # two outside: the copies fetch rows of zero points
    (1, 64, 6, 6, 32, 3, 1, (1, 1), (1, 0)),
    (1, 64, 6, 6, 32, 1, 3, (1, 1), (0, 1)),
    (24, 16, 56, 56, 32, 3, 3, (1, 1), (1, 1)),   # more pixel tiles than resident work-groups: each walks over several
]


@pytest.mark.parametrize("case", PADDED_WINDOWS)
@pytest.mark.parametrize("xdt", [np.uint8, np.int8])
def test_padding_with_any_zero_point(g, oracle, case, xdt):
    """Taps outside the image count as the activation zero point.  The matrix-core kernel fetches them as zeros and,
    for a zero point that is not the byte 0, starts each pixel's accumulators from what those zeros miss (windows that
    leave the image by at most one row or column per side); QLinearConv and ConvInteger against the oracle for zero
    points at both ends and inside the range, every tile shape on one of the cases."""
    import os
    N, C, H, W, OC, KH, KW, strides, pads = case
    rng = np.random.default_rng(41)
    x, w, ws, wz, bias, ys = make_case(rng, N, C, H, W, OC, KH, KW, xdt)
    zps = (0, 1, 128, 255) if xdt == np.uint8 else (-128, -1, 0, 5, 127)
    big = N * H * W > 10000
    if big:
        zps = zps[1:3]
        oracle.set_threads(16)
    xd = g.to_channels_last(g.dev(x))
    plan = g.ops.QLinearConvPlan(g.dev(w), g.dev(ws), g.dev(wz), g.dev(bias), strides=strides, pads=pads)
    try:
        for zp in zps:
            want = oracle.qlinear_conv_int(x, 0.02, zp, w, ws, wz, ys, 128, np.uint8, bias=bias, strides=strides, pads=pads,
                                           bias_mode=oracle.BIAS_ONNX_INT32)
            got = plan.run(xd, 0.02, zp, ys, 128, torch.uint8, flags=g.capi.BIAS_ONNX_INT32)
            np.testing.assert_array_equal(g.host(got), want, err_msg="zero point %d" % zp)
            if not big:
                want_int = oracle.conv_integer(x, w, zp, None, strides=strides, pads=pads)
                np.testing.assert_array_equal(g.host(g.ops.ConvInteger(xd, g.dev(w), zp, None, strides=strides, pads=pads)), want_int,
                                              err_msg="ConvInteger, zero point %d" % zp)
    finally:
        plan.close()
        oracle.set_threads(1)
    if case != PADDED_WINDOWS[3]:
        return
    zp = zps[1]
    want = oracle.qlinear_conv_int(x, 0.02, zp, w, ws, wz, ys, 128, np.uint8, bias=bias, strides=strides, pads=pads,
                                   bias_mode=oracle.BIAS_ONNX_INT32)
    before = os.environ.get("CHX_HIP_TILE")
    try:
        for tile in ("128,128,0,4", "128,64,0,4", "64,128,0,4", "64,64,0,4", "128,128,0,8", "128,256,0,8", "64,128,0,8"):
            os.environ["CHX_HIP_TILE"] = tile
            plan = g.ops.QLinearConvPlan(g.dev(w), g.dev(ws), g.dev(wz), g.dev(bias), strides=strides, pads=pads)
            got = plan.run(xd, 0.02, zp, ys, 128, torch.uint8, flags=g.capi.BIAS_ONNX_INT32)
            plan.close()
            np.testing.assert_array_equal(g.host(got), want, err_msg="tile %s" % tile)
    finally:
        if before is None:
            os.environ.pop("CHX_HIP_TILE", None)
        else:
            os.environ["CHX_HIP_TILE"] = before
