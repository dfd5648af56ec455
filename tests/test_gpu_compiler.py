"""ONNX graphs through the compiler side (quantizer, fusion, emitter) and the C++ VM on the MI355X,
compared with the CPU oracle: bit-exact for the 8-bit results and for the fused fp32 chain."""
import numpy as np
import pytest
import torch

import test_compiler_cpu as cc

pytestmark = pytest.mark.gpu
onnx_lite = cc.onnx_lite


@pytest.fixture(scope="module")
def g():
    import gpu_util
    gpu_util.capi.init(0)
    return gpu_util


@pytest.fixture(scope="module")
def vm(g):
    from importlib import import_module
    return import_module(g.pkg.__name__ + ".chxvm")


CHAIN = [("Mul", ["x", "a"], ["t0"]), ("Add", ["t0", "b"], ["t1"]), ("Tanh", ["t1"], ["t2"]), ("Sigmoid", ["c"], ["t3"]),
         ("Mul", ["t2", "t3"], ["t4"]), ("Add", ["t4", "x"], ["t5"]), ("Relu", ["t5"], ["y"])]
ORACLE_CHAIN = [("t0", "Mul", "x", "a"), ("t1", "Add", "t0", "b"), ("t2", "Tanh", "t1"), ("t3", "Sigmoid", "c"),
                ("t4", "Mul", "t2", "t3"), ("t5", "Add", "t4", "x"), ("y", "Relu", "t5")]


def test_float_chain_fused_and_op_by_op(g, vm, oracle):
    """relu(tanh(x*a+b)*sigmoid(c)+x): as one hip group, as the reference's group plus a lone Relu,
    and as seven single instructions -- the same bits each time, the oracle's."""
    rng = np.random.default_rng(11)
    shape = (6, 50, 128)
    x, c = rng.standard_normal(shape).astype(np.float32), rng.standard_normal(shape).astype(np.float32)
    a, b = rng.standard_normal(128).astype(np.float32), rng.standard_normal(128).astype(np.float32)
    want = oracle.run_chain(ORACLE_CHAIN, dict(x=x, a=a, b=b, c=c))["y"]
    m = cc.model(CHAIN, [("x", shape), ("a", (128,)), ("b", (128,)), ("c", shape)], [("y", shape)])
    counts = {}
    for fuse in ("hip", "nvrtc", "none"):
        data = vm.compile_onnx(m, {"fuse": fuse})
        names = [i[0] for i in cc.decode_program(vm, data)]
        counts[fuse] = (names.count("ElementWiseNvrtc"), names.count("Relu"), names.count("Mul"))
        prog = vm.Program(data)
        got = prog.run({k: torch.from_numpy(v).cuda() for k, v in dict(x=x, a=a, b=b, c=c).items()})["y"]
        prog.close()
        np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32), err_msg=fuse)
    assert counts == {"hip": (1, 0, 0), "nvrtc": (1, 1, 0), "none": (0, 1, 2)}


@pytest.mark.parametrize("per_channel,int8_weights", [(True, True), (False, True), (False, False), (True, False)])
def test_quantized_convolution_from_a_float_graph(g, vm, oracle, per_channel, int8_weights):
    """Conv -> (quantizer, static QLinearOps) -> QuantizeLinear, QLinearConv, DequantizeLinear, run on
    the device: equal to the oracle's ops applied to weights quantized by the numpy restatement."""
    rng = np.random.default_rng(12)
    m, w = cc.conv_model(rng)
    x = rng.standard_normal((1, 4, 8, 8)).astype(np.float32)
    opts = {"quantize": {"mode": "QLinearOps", "static": True, "asymmetric_input_types": int8_weights, "per_channel": per_channel,
                         "inputs": {"x": {"scale": 0.03, "zero_point": 121}}, "outputs": {"y": {"scale": 0.11, "zero_point": 90}}}}
    prog = vm.Program(vm.compile_onnx(m, opts))
    got = prog.run({"x": torch.from_numpy(x).cuda()})["y"]
    prog.close()
    wdt = np.int8 if int8_weights else np.uint8
    if per_channel:
        parts = [cc.numpy_quantize(w[c], wdt) for c in range(w.shape[0])]
        wq = np.stack([p[0] for p in parts])
        ws, wz = np.array([p[1] for p in parts], np.float32), np.array([p[2] for p in parts]).astype(wdt)
    else:
        wq, s, z = cc.numpy_quantize(w, wdt)
        ws, wz = np.float32(s), np.array(z).astype(wdt)
    xq = oracle.quantize_linear(x, 0.03, 121, np.uint8)
    yq = oracle.qlinear_conv_int(xq, 0.03, 121, wq, ws, wz, np.float32(0.11), 90, np.uint8, strides=(2, 2), pads=(1, 1))
    want = oracle.dequantize_linear(yq, 0.11, 90)
    assert len(np.unique(yq)) > 8
    np.testing.assert_array_equal(got, want)


def test_network_from_an_onnx_qdq_graph(g, vm, oracle):
    """The reduced ResNet written as an ONNX QDQ graph: the fusion pass turns every
    DequantizeLinear, DequantizeLinear, Add, Relu, QuantizeLinear run into one hip group, the emitter
    writes their parameters into the program text, and the VM computes each group inside the
    convolution before it; the logits are the oracle's."""
    wl = g.pkg.workloads
    model = wl.build_resnet50(batch=2, image=64, seed=5, width=16, blocks=(2, 1, 1, 1), classes=10)
    m = wl.program_to_onnx(model, onnx_lite)
    _, desc = vm.transform_onnx(m, {"fuse": "hip"})
    groups = [l for l in desc.splitlines() if l.startswith("ChainerFusionGroup")]
    assert len(groups) == 5 and all(l.endswith(": DequantizeLinear DequantizeLinear Add Relu QuantizeLinear]") or
                                    sorted(l.split(": ")[1].rstrip("]").split()) ==
                                    sorted("DequantizeLinear DequantizeLinear Add Relu QuantizeLinear".split()) for l in groups)
    data = vm.compile_onnx(m, {"fuse": "hip"})
    before = vm.counter("qlinearconv_residual_fusions")
    vm.set_option("qlinearconv_bias", "onnx_int32")
    try:
        prog = vm.Program(data)
        got = prog.run({"x": torch.from_numpy(model["input"]).cuda()})["logits"]
        prog.close()
    finally:
        vm.set_option("qlinearconv_bias", "reference")
    assert vm.counter("qlinearconv_residual_fusions") - before == 5
    oracle.set_threads(16)
    try:
        ref = wl.run_reference(model, oracle, model["input"], keep={"logits"})
    finally:
        oracle.set_threads(1)
    np.testing.assert_array_equal(got, ref["logits"])


def _dynamic_uint8_params(x):
    """The run-time parameter graph of the quantizer for a uint8 operand (compiler/quantize.cc:165-196),
    in float32 numpy operations: the range is NOT widened to contain 0 here."""
    rmin, rmax = np.float32(x.min()), np.float32(x.max())
    scale = np.float32(np.float32(rmax - rmin) / np.float32(255))
    zp = np.uint8(np.floor(np.float32(np.float32(0) - rmin) / scale))
    return scale, zp


@pytest.mark.parametrize("per_channel", [False, True])
def test_dynamic_integer_quantization_runs_end_to_end(g, vm, oracle, per_channel):
    """The reference's --quantize path (dynamic parameters, integer ops): ReduceMin/ReduceMax, the scalar
    arithmetic, QuantizeLinear, ConvInteger / MatMulInteger, Cast and the scale-back Mul all run on
    the device; the result equals the same sequence spelled with numpy and the oracle."""
    rng = np.random.default_rng(13)
    m, w = cc.conv_model(rng)
    x = (rng.standard_normal((1, 4, 8, 8)) * 2 + 0.3).astype(np.float32)
    prog = vm.Program(vm.compile_onnx(m, {"quantize": {"per_channel": per_channel}}))
    got = prog.run({"x": torch.from_numpy(x).cuda()})["y"]
    prog.close()
    scale, zp = _dynamic_uint8_params(x)
    xq = oracle.quantize_linear(x, scale, int(zp), np.uint8)
    if per_channel:
        parts = [cc.numpy_quantize(w[c], np.uint8) for c in range(w.shape[0])]
        wq = np.stack([p[0] for p in parts])
        ws, wz = np.array([p[1] for p in parts], np.float32), np.array([p[2] for p in parts], np.uint8)
    else:
        wq, s, z = cc.numpy_quantize(w, np.uint8)
        ws, wz = np.float32(s), np.array(z, np.uint8)
    acc = oracle.conv_integer(xq, wq, int(zp), wz, strides=(2, 2), pads=(1, 1), group=1, auto_pad="")
    scales = (scale * ws).astype(np.float32)
    want = acc.astype(np.float32) * (scales.reshape(-1, 1, 1) if per_channel else scales)
    np.testing.assert_array_equal(got, want.astype(np.float32))
    # the quantized result tracks the float convolution
    ref = torch.nn.functional.conv2d(torch.from_numpy(x), torch.from_numpy(w), stride=2, padding=1).numpy()
    assert np.abs(got - ref).max() < 0.05 * np.abs(ref).max() + 0.05
    # MatMul the same way
    b = rng.standard_normal((5, 3)).astype(np.float32)
    a = rng.standard_normal((4, 5)).astype(np.float32)
    mm = cc.model([("MatMul", ["a", "b"], ["y"])], [("a", (4, 5))], [("y", (4, 3))], {"b": b})
    prog = vm.Program(vm.compile_onnx(mm, {"quantize": {}}))
    got = prog.run({"a": torch.from_numpy(a).cuda()})["y"]
    prog.close()
    sa, za = _dynamic_uint8_params(a)
    bq, sb, zb = cc.numpy_quantize(b, np.uint8)
    acc = oracle.matmul_integer(oracle.quantize_linear(a, sa, int(za), np.uint8), bq, np.array(za, np.uint8), np.array(zb, np.uint8))
    np.testing.assert_array_equal(got, acc.astype(np.float32) * np.float32(sa * sb))


def test_clip_round_and_friends_as_single_instructions(g, vm):
    """Clip with attribute bounds (StaticClip), Clip with operand bounds, one bound missing, Round
    (ties to even), Abs, Floor, Max and Min as instructions of their own and inside one hip group:
    the bytes numpy gives for the same float32 operations."""
    rng = np.random.default_rng(14)
    x = np.concatenate([rng.uniform(-9, 9, 500).astype(np.float32),
                        np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 6.0, -3.0, 0.0], np.float32)]).reshape(1, 509)
    f32 = np.float32
    lo = onnx_lite.Node("Constant", [], ["lo"], {"value": np.array(-2.25, f32)})
    hi = onnx_lite.Node("Constant", [], ["hi"], {"value": np.array(5.5, f32)})
    nodes = [lo, hi,
             onnx_lite.Node("Clip", ["x"], ["a"], {"min": -3.0, "max": 6.0}),       # bounds as attributes
             onnx_lite.Node("Clip", ["x", "lo", "hi"], ["b"]),                       # bounds as operands
             onnx_lite.Node("Clip", ["x", "", "hi"], ["c"]),                         # no lower bound
             ("Round", ["x"], ["d"]), ("Abs", ["x"], ["e"]), ("Floor", ["x"], ["f"]),
             ("Max", ["a", "d"], ["m"]), ("Min", ["b", "f"], ["n"])]
    outs = ["a", "b", "c", "d", "e", "f", "m", "n"]
    m = cc.model(nodes, [("x", x.shape)], [(o, x.shape) for o in outs])
    a, b, c = np.clip(x, f32(-3), f32(6)), np.clip(x, f32(-2.25), f32(5.5)), np.minimum(x, f32(5.5))
    d, e, f = np.rint(x), np.abs(x), np.floor(x)
    want = dict(a=a, b=b, c=c, d=d, e=e, f=f, m=np.maximum(a, d), n=np.minimum(b, f))
    assert d[0, -9:].tolist() == [0.0, 2.0, 2.0, -0.0, -2.0, -2.0, 6.0, -3.0, 0.0]
    for fuse in ("none", "hip"):
        data = vm.compile_onnx(m, {"fuse": fuse})
        names = [i[0] for i in cc.decode_program(vm, data)]
        if fuse == "none":
            assert names.count("StaticClip") == 1 and names.count("Clip") == 2 and "Round" in names
        prog = vm.Program(data)
        got = prog.run({"x": torch.from_numpy(x).cuda()})
        prog.close()
        for o in outs:
            np.testing.assert_array_equal(got[o].view(np.uint32), want[o].view(np.uint32), err_msg="%s (%s)" % (o, fuse))
