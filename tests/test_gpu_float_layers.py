"""The float32 layers around a quantized network: Gemm, Linear, MatMul, Flatten (runtime/ops/math.cc:156-177,
runtime/ops/connection.cc:12-15, runtime/ops/manipulation.cc:20-28 of the chainer-compiler tree), through
the C ABI and as instructions of a serialized program.  The device sums in the oracle's order (ascending
k, one rounding per operation), so results are compared bit for bit; against a float64 product the bar
is the bound of a float32 sum of K terms."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def g():
    import gpu_util
    gpu_util.capi.init(0)
    return gpu_util


@pytest.fixture(scope="module")
def vm(g):
    from importlib import import_module
    return import_module(g.pkg.__name__ + ".chxvm")


def bits(a):
    return np.ascontiguousarray(a).view(np.int32)


GEMM_CASES = [
    # M, N, K, trans_a, trans_b, c shape (None: no c), alpha, beta
    (32, 100, 784, False, False, None, 1.0, 1.0),          # the MLP of the reference's quantization test, first layer
    (32, 10, 100, False, True, (10,), 1.0, 1.0),           # the Linear route of GemmOp
    (64, 1000, 2048, False, True, (1000,), 1.0, 1.0),      # ResNet-50 classifier at batch 64
    (7, 5, 3, True, False, (7, 1), 0.5, 2.0),
    (65, 129, 17, True, True, (65, 129), 1.0, -1.0),
    (1, 1, 1, False, False, (1, 1), 3.0, 1.0),
    (130, 66, 300, False, False, (1, 66), 1.0, 0.0),       # beta == 0: c is not read
    (3, 4, 0, False, False, (4,), 1.0, 1.0),               # an empty sum is 0
]


@pytest.mark.parametrize("case", GEMM_CASES, ids=lambda c: "M%d_N%d_K%d_%s%s" % (c[0], c[1], c[2], "T" if c[3] else "N", "T" if c[4] else "N"))
def test_gemm_through_the_c_abi(g, oracle, case):
    M, N, K, ta, tb, cshape, alpha, beta = case
    rng = np.random.default_rng(M * 1000 + N)
    a = rng.standard_normal((K, M) if ta else (M, K)).astype(np.float32)
    b = rng.standard_normal((N, K) if tb else (K, N)).astype(np.float32)
    c = None if cshape is None else rng.standard_normal(cshape).astype(np.float32)
    if beta == 0.0 and c is not None:
        c[...] = np.nan
    want = oracle.gemm(a, b, c, alpha, beta, ta, tb)
    got = g.host(g.ops.Gemm(g.dev(a), g.dev(b), None if c is None else g.dev(c), alpha, beta, int(ta), int(tb)))
    assert got.shape == (M, N) and got.dtype == np.float32
    np.testing.assert_array_equal(bits(got), bits(want))
    if K:
        A, B = (a.T if ta else a).astype(np.float64), (b.T if tb else b).astype(np.float64)
        exact = alpha * (A @ B) + (0 if c is None or beta == 0.0 else beta * c.astype(np.float64))
        bound = (K + 3) * 2.0 ** -24 * (abs(alpha) * (np.abs(A) @ np.abs(B)) + (0 if c is None or beta == 0.0 else np.abs(beta * c)))
        assert (np.abs(got - exact) <= bound + 1e-30).all()


def test_gemm_reads_operands_through_their_strides(g, oracle):
    rng = np.random.default_rng(7)
    big_a = rng.standard_normal((40, 90)).astype(np.float32)
    big_b = rng.standard_normal((90, 50)).astype(np.float32)
    a, b = big_a[3:33:2, 5:65:3], big_b[10:30, ::5]      # 15 x 20 and 20 x 10 views
    da, db = g.dev(big_a)[3:33:2, 5:65:3], g.dev(big_b)[10:30, ::5]
    out = torch.zeros((15, 30), dtype=torch.float32, device="cuda")[:, ::3]
    g.ops.Gemm(da, db, out=out)
    np.testing.assert_array_equal(bits(g.host(out)), bits(oracle.gemm(np.ascontiguousarray(a), np.ascontiguousarray(b))))
    # a transposed view is the transposed operand
    np.testing.assert_array_equal(bits(g.host(g.ops.Gemm(da.t(), db.t(), trans_a=1, trans_b=1))),
                                  bits(oracle.gemm(np.ascontiguousarray(a), np.ascontiguousarray(b))))


def test_gemm_refuses_what_it_cannot_compute(g):
    a, b = g.dev(np.zeros((3, 4), np.float32)), g.dev(np.zeros((5, 6), np.float32))
    with pytest.raises(g.capi.ChxHipError, match="inner extents"):
        g.ops.Gemm(a, b)
    with pytest.raises(g.capi.ChxHipError, match="float32"):
        g.ops.Gemm(a, g.dev(np.zeros((4, 6), np.int32)))
    with pytest.raises(g.capi.ChxHipError, match="broadcast"):
        g.ops.Gemm(a, g.dev(np.zeros((4, 6), np.float32)), g.dev(np.zeros((5,), np.float32)))


def test_linear_over_batch_axes(g, oracle):
    rng = np.random.default_rng(9)
    x = rng.standard_normal((2, 3, 4, 5)).astype(np.float32)
    for nb, k in ((1, 60), (2, 20), (3, 5)):
        w = rng.standard_normal((7, k)).astype(np.float32)
        bias = rng.standard_normal((7,)).astype(np.float32)
        got = g.host(g.ops.Linear(g.dev(x), g.dev(w), g.dev(bias), nb))
        assert got.shape == x.shape[:nb] + (7,)
        np.testing.assert_array_equal(bits(got), bits(oracle.linear(x, w, bias, nb)))
        np.testing.assert_array_equal(bits(g.host(g.ops.Linear(g.dev(x), g.dev(w), None, nb))), bits(oracle.linear(x, w, None, nb)))
    with pytest.raises(g.capi.ChxHipError, match="n_batch_axes"):
        g.ops.Linear(g.dev(x), g.dev(np.zeros((7, 5), np.float32)), None, 4)


def test_flatten(g, oracle):
    x = np.arange(2 * 3 * 4 * 5).reshape(2, 3, 4, 5).astype(np.float32)
    for axis in (0, 1, 2, 3, -1, -3):
        np.testing.assert_array_equal(g.host(g.ops.Flatten(g.dev(x), axis)), oracle.flatten(x, axis))
    # a channels-last tensor flattens in its logical (NCHW) order
    np.testing.assert_array_equal(g.host(g.ops.Flatten(g.to_channels_last(g.dev(x)), 1)), x.reshape(2, 60))
    q = np.arange(2 * 16 * 3 * 3).reshape(2, 16, 3, 3).astype(np.uint8)
    np.testing.assert_array_equal(g.host(g.ops.Flatten(g.to_channels_last(g.dev(q)), 1)), q.reshape(2, 144))
    with pytest.raises(ValueError):
        g.ops.Flatten(g.dev(x), 4)


POOL_SHAPES = [
    # N, C, H, W, kernel, strides, pads
    (2, 16, 13, 12, (3, 3), (2, 2), (0, 0)), (1, 5, 9, 9, (2, 2), (2, 2), (1, 1)), (2, 3, 7, 7, (7, 7), (1, 1), (0, 0)),
    (1, 4, 11, 10, (4, 5), (2, 3), (1, 2)), (3, 2, 6, 6, (1, 1), (2, 2), (0, 0)), (64, 8, 28, 28, (3, 3), (2, 2), (1, 1)),
]


@pytest.mark.parametrize("case", POOL_SHAPES, ids=lambda c: "x".join(str(v) for v in c[:4]) + "_k%dx%d" % c[4])
def test_float_pools_through_the_c_abi(g, oracle, case):
    """MaxPool (both cover_all settings) and AveragePool (both pad-count modes) on float32, NCHW and channels-last,
    bit for bit against the oracle (the sum of a window is taken in the oracle's order)."""
    N, C, H, W, kernel, strides, pads = case
    rng = np.random.default_rng(H * 100 + W)
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    for xd in (g.dev(x), g.to_channels_last(g.dev(x))):
        for cover_all in (False, True):
            got = g.host(g.ops.MaxPool(xd, kernel, strides, pads, cover_all))
            np.testing.assert_array_equal(got, oracle.max_pool(x, kernel, strides, pads, cover_all))
        for include_pad in (False, True):
            got = g.host(g.ops.AveragePool(xd, kernel, strides, pads, include_pad))
            np.testing.assert_array_equal(bits(got), bits(oracle.average_pool(x, kernel, strides, pads, include_pad)))
    with pytest.raises(g.capi.ChxHipError, match="float32"):
        g.ops.MaxPool(g.dev(np.zeros((1, 1, 4, 4), np.uint8)), (2, 2), out=torch.zeros((1, 1, 3, 3), dtype=torch.float32, device="cuda"))


def test_float_layers_as_program_instructions(g, vm, oracle):
    """Flatten -> Gemm (Linear route) -> Relu -> MatMul -> Linear in one serialized program, against the
    oracle op by op."""
    rng = np.random.default_rng(11)
    x = rng.standard_normal((4, 8, 3, 3)).astype(np.float32)
    w1 = rng.standard_normal((20, 72)).astype(np.float32)
    b1 = rng.standard_normal((20,)).astype(np.float32)
    w2 = rng.standard_normal((20, 6)).astype(np.float32)
    w3 = rng.standard_normal((5, 6)).astype(np.float32)
    b = vm.ProgramBuilder()
    xs = b.input("x", "float32", x.shape)
    f = b.Flatten(xs, 1)
    h = b.Gemm(f, b.constant(w1), b.constant(b1), 1.0, 1.0, 0, 1)
    r = b.Relu(h)
    m = b.MatMul(r, b.constant(w2))
    y = b.Linear(m, b.constant(w3), None, 1)
    g2 = b.Gemm(r, b.constant(w2), None, 0.25, 1.0, 0, 0)
    for name, slot in (("f", f), ("h", h), ("m", m), ("y", y), ("g2", g2)):
        b.output(name, slot)
    prog = vm.Program(b.serialize())
    want_f = oracle.flatten(x, 1)
    want_h = oracle.gemm(want_f, w1, b1, trans_b=True)
    want_r = np.maximum(want_h, np.float32(0))
    want_m = oracle.gemm(want_r, w2)
    want_y = oracle.linear(want_m, w3)
    for xd in (g.dev(x), g.to_channels_last(g.dev(x))):     # a channels-last input is copied dense by Flatten
        out = prog.run({"x": xd})
        np.testing.assert_array_equal(out["f"], want_f)
        np.testing.assert_array_equal(bits(out["h"]), bits(want_h))
        np.testing.assert_array_equal(bits(out["m"]), bits(want_m))
        np.testing.assert_array_equal(bits(out["y"]), bits(want_y))
        np.testing.assert_array_equal(bits(out["g2"]), bits(oracle.gemm(want_r, w2, alpha=0.25)))
    prog.close()


def test_float_layers_from_an_onnx_graph(g, vm, oracle):
    """Flatten, Gemm and MatMul nodes of an ONNX graph reach the VM through the compiler's emitter."""
    import test_compiler_cpu as cc
    rng = np.random.default_rng(12)
    x = rng.standard_normal((3, 2, 4, 4)).astype(np.float32)
    w = rng.standard_normal((9, 32)).astype(np.float32)
    bias = rng.standard_normal((9,)).astype(np.float32)
    w2 = rng.standard_normal((9, 4)).astype(np.float32)
    N = cc.onnx_lite.Node
    m = cc.model([N("Flatten", ["x"], ["f"], {"axis": 1}), N("Gemm", ["f", "w", "b"], ["h"], {"transB": 1}), N("MatMul", ["h", "w2"], ["y"], {})],
                 [("x", x.shape)], [("y", (3, 4))], {"w": w, "b": bias, "w2": w2})
    prog = vm.Program(vm.compile_onnx(m, {"fuse": "none"}))
    got = prog.run({"x": g.dev(x)})
    prog.close()
    want = oracle.gemm(oracle.gemm(oracle.flatten(x, 1), w, bias, trans_b=True), w2)
    np.testing.assert_array_equal(bits(got["y"]), bits(want))


@pytest.mark.parametrize("shape", [(4, 6, 5, 7), (2, 16, 14, 14), (3, 5), (2, 4, 9), (1, 1, 1, 1)], ids=str)
def test_fixed_batch_norm_through_the_c_abi(g, oracle, shape):
    """FixedBatchNormalization on NCHW, channels-last, [N, C] and [N, C, L] arrays, bit for bit against the oracle
    (square root and reciprocal are correctly rounded on both sides); epsilon at or below 1e-5 is replaced."""
    rng = np.random.default_rng(sum(shape))
    C = shape[1]
    x = (rng.standard_normal(shape) * 3).astype(np.float32)
    s, bias, mean = (rng.standard_normal(C).astype(np.float32) for _ in range(3))
    var = rng.uniform(0.0, 4.0, C).astype(np.float32)
    for eps in (1e-3, 1e-5, 0.0):
        want = oracle.fixed_batch_norm(x, s, bias, mean, var, eps)
        layouts = [g.dev(x)] + ([g.to_channels_last(g.dev(x))] if len(shape) == 4 else [])
        for xd in layouts:
            got = g.ops.FixedBatchNormalization(xd, g.dev(s), g.dev(bias), g.dev(mean), g.dev(var.reshape(1, C)), eps)
            assert got.stride() == xd.stride()
            np.testing.assert_array_equal(bits(g.host(got)), bits(want))
    with pytest.raises(g.capi.ChxHipError, match="channels"):
        g.ops.FixedBatchNormalization(g.dev(x), g.dev(s[:-1] if C > 1 else np.zeros(2, np.float32)), g.dev(bias), g.dev(mean), g.dev(var))
    with pytest.raises(g.capi.ChxHipError, match="float32"):
        g.ops.FixedBatchNormalization(g.dev(x.astype(np.float64)).to(torch.float64), g.dev(s), g.dev(bias), g.dev(mean), g.dev(var),
                                      out=torch.empty(shape, dtype=torch.float32, device="cuda"))


FCONV_CASES = [  # N, C, H, W, OC, KH, KW, strides, pads, group, auto_pad
    (2, 3, 9, 8, 4, 3, 3, (1, 1), (1, 1), 1, ""), (1, 4, 7, 7, 6, 1, 1, (2, 2), (0, 0), 2, ""), (2, 6, 8, 8, 6, 3, 2, (2, 1), (0, 1), 6, ""),
    (1, 8, 5, 5, 4, 5, 5, (1, 1), (2, 2), 4, ""), (3, 2, 6, 6, 5, 2, 2, (2, 2), (0, 0), 1, ""), (2, 16, 14, 14, 32, 3, 3, (2, 2), (0, 0), 1, "SAME_UPPER"),
    (4, 3, 32, 32, 16, 7, 7, (2, 2), (3, 3), 1, "")]


@pytest.mark.parametrize("case", FCONV_CASES, ids=lambda c: "x".join(str(v) for v in c[:7]) + "_g%d" % c[9])
def test_float_conv_through_the_c_abi(g, oracle, case):
    """The float32 Conv the quantizer leaves alone (one with a bias): NCHW and channels-last, with and without the bias,
    groups, strides, pads and SAME_UPPER; bit for bit against the oracle, whose order of the sum the kernel follows."""
    N, C, H, W, OC, KH, KW, strides, pads, group, auto_pad = case
    rng = np.random.default_rng(N * 100 + C * 10 + KH)
    x = rng.standard_normal((N, C, H, W)).astype(np.float32)
    w = rng.standard_normal((OC, C // group, KH, KW)).astype(np.float32)
    b = rng.standard_normal(OC).astype(np.float32)
    for bias in (b, None):
        want = oracle.conv(x, w, bias, strides, pads, group, auto_pad)
        for xd in (g.dev(x), g.to_channels_last(g.dev(x))):
            got = g.ops.Conv(xd, g.dev(w), None if bias is None else g.dev(bias), strides, pads, group, auto_pad)
            assert got.shape == want.shape
            np.testing.assert_array_equal(bits(g.host(got)), bits(want))
    with pytest.raises(g.capi.ChxHipError, match="float32"):
        g.ops.Conv(g.dev(x), g.dev(w.astype(np.float64)).to(torch.float64), None, strides, pads, group, auto_pad)


def test_conv_net_with_batch_normalization_under_the_default_quantization(g, vm, oracle):
    """What `--quantize` (dynamic parameters, integer ops) leaves of a float CNN: the Conv without a bias becomes
    QuantizeLinear -> ConvInteger -> Cast -> Mul, and the Conv with a bias, BatchNormalization, Relu, MaxPool,
    GlobalAveragePool, Flatten and Gemm stay float nodes (compiler/quantize.cc:377-380, compiler/chxvm/emitter.cc:193-206).  The program is compared with
    the same sequence spelled with numpy and the oracle, and loosely with the float network."""
    import test_compiler_cpu as cc
    import test_gpu_compiler as gc
    onnx_lite = cc.onnx_lite
    rng = np.random.default_rng(21)
    N = onnx_lite.Node
    w = (rng.standard_normal((8, 3, 3, 3)) * 0.3).astype(np.float32)
    s, bias, mean = (rng.standard_normal(8).astype(np.float32) * 0.5 for _ in range(3))
    s = s + np.float32(1.5)
    var = rng.uniform(0.5, 2.0, 8).astype(np.float32)
    w2 = (rng.standard_normal((8, 8, 3, 3)) * 0.2).astype(np.float32)
    b2 = rng.standard_normal(8).astype(np.float32)
    fc = (rng.standard_normal((5, 8)) * 0.4).astype(np.float32)
    fb = rng.standard_normal(5).astype(np.float32)
    nodes = [N("Conv", ["x", "w"], ["c"], {"kernel_shape": [3, 3], "strides": [1, 1], "pads": [1, 1, 1, 1]}),
             N("BatchNormalization", ["c", "s", "bias", "mean", "var"], ["bn"], {"epsilon": 1e-5}),
             N("Relu", ["bn"], ["r0"], {}),
             N("Conv", ["r0", "w2", "b2"], ["r"], {"kernel_shape": [3, 3], "pads": [1, 1, 1, 1]}),       # with a bias: not rewritten
             N("MaxPool", ["r"], ["p"], {"kernel_shape": [2, 2], "strides": [2, 2]}),
             N("GlobalAveragePool", ["p"], ["ga"], {}),
             N("Flatten", ["ga"], ["f"], {}),
             N("Gemm", ["f", "fc", "fb"], ["y"], {"transB": 1})]
    x = (rng.standard_normal((2, 3, 12, 12)) * 1.5).astype(np.float32)
    m = cc.model(nodes, [("x", x.shape)], [("y", (2, 5))], {"w": w, "s": s, "bias": bias, "mean": mean, "var": var, "fc": fc, "fb": fb, "w2": w2, "b2": b2},
                 value_info=[("p", (2, 8, 6, 6))])
    data = vm.compile_onnx(m, {"quantize": {}})
    names = [i[0] for i in cc.decode_program(vm, data)]
    assert names.count("ConvInteger") == 1 and names.count("Conv") == 1 and "FixedBatchNormalization" in names and "Gemm" in names
    prog = vm.Program(data)
    got = prog.run({"x": torch.from_numpy(x).cuda()})["y"]
    prog.close()
    scale, zp = gc._dynamic_uint8_params(x)
    xq = oracle.quantize_linear(x, scale, int(zp), np.uint8)
    parts = [cc.numpy_quantize(w[oc], np.uint8) for oc in range(w.shape[0])]     # per output channel: the quantizer's default
    wq = np.stack([q[0] for q in parts])
    ws, wz = np.array([q[1] for q in parts], np.float32), np.array([q[2] for q in parts], np.uint8)
    acc = oracle.conv_integer(xq, wq, int(zp), wz, strides=(1, 1), pads=(1, 1), group=1, auto_pad="")
    c = acc.astype(np.float32) * (scale * ws).astype(np.float32).reshape(-1, 1, 1)
    bn = oracle.fixed_batch_norm(c, s, bias, mean, var, 1e-5)
    r = oracle.conv(np.maximum(bn, np.float32(0)), w2, b2, (1, 1), (1, 1))
    p = oracle.max_pool(r, (2, 2), (2, 2), (0, 0), False)
    ga = oracle.average_pool(p, (6, 6), (1, 1), (0, 0), False)
    want = oracle.gemm(oracle.flatten(ga, 1), fc, fb, trans_b=True)
    np.testing.assert_array_equal(bits(got), bits(want))
    tx = torch.from_numpy
    ref = torch.nn.functional.conv2d(tx(x), tx(w), padding=1)
    ref = torch.nn.functional.batch_norm(ref, tx(mean), tx(var), tx(s), tx(bias), eps=1e-5).relu()
    ref = torch.nn.functional.conv2d(ref, tx(w2), tx(b2), padding=1)
    ref = torch.nn.functional.max_pool2d(ref, 2).mean(dim=(2, 3)) @ tx(fc).T + tx(fb)
    assert np.abs(got - ref.numpy()).max() < 0.05 * np.abs(ref.numpy()).max() + 0.05


@pytest.mark.parametrize("shape,axis", [((4, 10), 1), ((3, 5, 7), 1), ((3, 5, 7), 2), ((2, 3, 4, 5), 1), ((6,), 0), ((64, 1000), -1),
                                        ((2, 3, 4, 5), 0), ((1, 1), 1)], ids=str)
def test_softmax_through_the_c_abi(g, oracle, shape, axis):
    """Softmax with both axis semantics, bit for bit against the oracle (exp as the C library's expf on both sides)."""
    rng = np.random.default_rng(len(shape) * 10 + axis)
    x = (rng.standard_normal(shape) * 4).astype(np.float32)
    x.reshape(-1)[::7] *= 12          # arguments far below the maximum: exp underflows to denormals and to 0
    for onnx in (True, False):
        got = g.host(g.ops.Softmax(g.dev(x), axis, onnx))
        np.testing.assert_array_equal(bits(got), bits(oracle.softmax(x, axis, onnx)))
    with pytest.raises(g.capi.ChxHipError, match="axis"):
        g.ops.Softmax(g.dev(x), len(shape), True)


def test_softmax_from_an_onnx_graph(g, vm, oracle):
    """Gemm -> Softmax (the head of a classifier) through the emitter: attribute defaults axis = 1 and ONNX semantics,
    and an explicit axis 0 (everything reduced together)."""
    import test_compiler_cpu as cc
    rng = np.random.default_rng(31)
    x = rng.standard_normal((5, 12)).astype(np.float32)
    w = rng.standard_normal((12, 7)).astype(np.float32)
    N = cc.onnx_lite.Node
    m = cc.model([N("Gemm", ["x", "w"], ["h"], {}), N("Softmax", ["h"], ["y"], {}), N("Softmax", ["h"], ["z"], {"axis": 0})],
                 [("x", x.shape)], [("y", (5, 7)), ("z", (5, 7))], {"w": w})
    insts = cc.decode_program(vm, vm.compile_onnx(m, {"fuse": "none"}))
    assert [[v for _, v in i[1][1:]] for i in insts if i[0] == "Softmax"] == [[1, 1], [0, 1]]
    prog = vm.Program(vm.compile_onnx(m, {"fuse": "none"}))
    out = prog.run({"x": g.dev(x)})
    prog.close()
    h = oracle.gemm(x, w)
    np.testing.assert_array_equal(bits(out["y"]), bits(oracle.softmax(h, 1, True)))
    np.testing.assert_array_equal(bits(out["z"]), bits(oracle.softmax(h, 0, True)))


def test_views_between_the_float_layers(g, vm, oracle):
    """Transpose (a view, no perm = reversed axes), Squeeze (named axes, or every axis of extent 1) and Unsqueeze
    (runtime/ops/manipulation.cc:60-72, 101-107) as they occur between a pooled feature map and a classifier head:
    GlobalAveragePool -> Squeeze -> Gemm -> Transpose -> Softmax over the other axis -> Unsqueeze."""
    import test_compiler_cpu as cc
    rng = np.random.default_rng(41)
    N = cc.onnx_lite.Node
    x = rng.standard_normal((4, 6, 3, 5)).astype(np.float32)
    w = rng.standard_normal((6, 7)).astype(np.float32)
    nodes = [N("GlobalAveragePool", ["x"], ["p"], {}), N("Squeeze", ["p"], ["s"], {"axes": [2, 3]}), N("Squeeze", ["p"], ["s_all"], {}),
             N("Gemm", ["s", "w"], ["h"], {}), N("Transpose", ["h"], ["t"], {}), N("Softmax", ["t"], ["sm"], {"axis": 1}),
             N("Unsqueeze", ["sm"], ["u"], {"axes": [0, 3]}), N("Transpose", ["x"], ["xt"], {"perm": [0, 2, 3, 1]}),
             N("Unsqueeze", ["s_all"], ["u2"], {"axes": [-1]})]
    outs = [("s_all", (4, 6)), ("t", (7, 4)), ("u", (1, 7, 4, 1)), ("xt", (4, 3, 5, 6)), ("u2", (4, 6, 1))]
    m = cc.model(nodes, [("x", x.shape)], outs, {"w": w})
    prog = vm.Program(vm.compile_onnx(m, {"fuse": "none"}))
    out = prog.run({"x": g.dev(x)})
    prog.close()
    pooled = oracle.average_pool(x, (3, 5), (1, 1), (0, 0), False).reshape(4, 6)
    h = oracle.gemm(pooled, w)
    np.testing.assert_array_equal(out["s_all"], pooled)
    np.testing.assert_array_equal(bits(out["t"]), bits(np.ascontiguousarray(h.T)))
    np.testing.assert_array_equal(bits(out["u"]), bits(oracle.softmax(np.ascontiguousarray(h.T), 1, True).reshape(1, 7, 4, 1)))
    np.testing.assert_array_equal(out["xt"], x.transpose(0, 2, 3, 1))
    np.testing.assert_array_equal(out["u2"], pooled.reshape(4, 6, 1))
    bad = cc.model([N("Squeeze", ["x"], ["y"], {"axes": [1]})], [("x", x.shape)], [("y", (4, 3, 5))])
    prog = vm.Program(vm.compile_onnx(bad, {"fuse": "none"}))
    with pytest.raises(vm.ChxVMError, match="extent 6"):
        prog.run({"x": g.dev(x)})
    prog.close()


def test_concat_as_a_program_instruction(g, vm):
    """ConcatOp::RunImpl (runtime/ops/manipulation.cc:74-76): along the channel axis of NCHW and of channels-last feature
    maps, along the first and the last axis, float32 and uint8; inputs of different extents on the axis."""
    import test_compiler_cpu as cc
    rng = np.random.default_rng(51)
    N = cc.onnx_lite.Node
    a = rng.standard_normal((2, 3, 4, 5)).astype(np.float32)
    b = rng.standard_normal((2, 5, 4, 5)).astype(np.float32)
    c = rng.standard_normal((2, 1, 4, 5)).astype(np.float32)
    m = cc.model([N("Concat", ["a", "b", "c"], ["ch"], {"axis": 1}), N("Concat", ["a", "a"], ["n"], {"axis": 0}),
                  N("Concat", ["a", "a", "a"], ["w"], {"axis": -1})],
                 [("a", a.shape), ("b", b.shape), ("c", c.shape)], [("ch", (2, 9, 4, 5)), ("n", (4, 3, 4, 5)), ("w", (2, 3, 4, 15))])
    prog = vm.Program(vm.compile_onnx(m, {"fuse": "none"}))
    for lay in (g.dev, lambda t: g.to_channels_last(g.dev(t))):
        out = prog.run({"a": lay(a), "b": lay(b), "c": lay(c)})
        np.testing.assert_array_equal(out["ch"], np.concatenate([a, b, c], axis=1))
        np.testing.assert_array_equal(out["n"], np.concatenate([a, a], axis=0))
        np.testing.assert_array_equal(out["w"], np.concatenate([a, a, a], axis=3))
    prog.close()
    # codes: a builder program, since ONNX value infos of the test helper are float
    qa = rng.integers(0, 256, size=(1, 16, 3, 3)).astype(np.uint8)
    qb = rng.integers(0, 256, size=(1, 32, 3, 3)).astype(np.uint8)
    bld = vm.ProgramBuilder()
    sa, sb = bld.input("a", "uint8", qa.shape), bld.input("b", "uint8", qb.shape)
    y = bld.new_slot()
    bld.add_raw("Concat", [("ARRAY_LIST", [sa, sb]), ("INT", 1)], [y])
    bld.output("y", y)
    prog = vm.Program(bld.serialize())
    out = prog.run({"a": g.to_channels_last(g.dev(qa)), "b": g.to_channels_last(g.dev(qb))})
    np.testing.assert_array_equal(out["y"], np.concatenate([qa, qb], axis=1))
    with pytest.raises(vm.ChxVMError, match="extents differ"):
        prog.run({"a": g.dev(qa), "b": g.dev(qb[:, :, :2])})
    prog.close()
