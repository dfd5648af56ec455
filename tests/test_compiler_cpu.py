"""The compiler side without a GPU: ONNX reader/writer, graph IR, fusion-group formation, the hip
program builder, the quantizer pass and the emitter -- against the reference's own fusion test
(compiler/fusion_test.cc: Tanh -> Sigmoid becomes one group of two), against independent numpy
restatements of the weight quantization formulas (compiler/quantize.cc:68-89), and against the
rewrites that pass documents (node sequences, operand order, copied attributes)."""
import os
import sys

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
import __graft_entry__ as entry  # noqa: E402

pkg = entry.load_package()
from importlib import import_module  # noqa: E402

onnx_lite = import_module(pkg.__name__ + ".onnx_lite")
F = onnx_lite.FLOAT


@pytest.fixture(scope="module")
def vm():
    mod = import_module(pkg.__name__ + ".chxvm")
    if not os.path.exists(mod.RUNTIME_LIB):
        entry.build()
    mod.runtime()
    return mod


def model(nodes, inputs, outputs, initializers=None, value_info=()):
    g = onnx_lite.Graph()
    g.value_info = [(n, F, list(s)) for n, s in value_info]
    g.name = "test"
    g.nodes = [onnx_lite.Node(*n) if not isinstance(n, onnx_lite.Node) else n for n in nodes]
    g.inputs = [(n, F, list(s)) for n, s in inputs]
    g.outputs = [(n, F, list(s)) for n, s in outputs]
    g.initializers = dict(initializers or {})
    for name, a in g.initializers.items():
        g.inputs.append((name, onnx_lite.ONNX_OF[a.dtype], list(a.shape)))
    return onnx_lite.make_model(g)


def lines(desc):
    return [l for l in desc.splitlines() if l]


def ops_of(desc):
    return [l.split("(")[0] for l in lines(desc)]


def test_fusion_basic_tanh_sigmoid(vm):
    """compiler/fusion_test.cc:11-30."""
    m = model([("Tanh", ["input"], ["tmp"]), ("Sigmoid", ["tmp"], ["output"])], [("input", ())], [("output", ())])
    for kind in ("nvrtc", "hip"):
        _, desc = vm.transform_onnx(m, {"fuse": kind})
        assert len(lines(desc)) == 1
        assert lines(desc)[0].startswith("ChainerFusionGroup(input) -> (output)")
        assert lines(desc)[0].endswith("[%s #1: Tanh Sigmoid]" % kind)
    _, desc = vm.transform_onnx(m, {"fuse": "none"})
    assert ops_of(desc) == ["Tanh", "Sigmoid"]


def test_fusable_sets_and_minimum_size(vm):
    chain = [("Mul", ["x", "a"], ["t0"]), ("Add", ["t0", "b"], ["t1"]), ("Tanh", ["t1"], ["t2"]), ("Sigmoid", ["c"], ["t3"]),
             ("Mul", ["t2", "t3"], ["t4"]), ("Add", ["t4", "x"], ["t5"]), ("Relu", ["t5"], ["y"])]
    m = model(chain, [("x", (4, 8)), ("a", (8,)), ("b", (8,)), ("c", (4, 8))], [("y", (4, 8))])
    # the reference's set has no Relu: it stays outside the group
    _, desc = vm.transform_onnx(m, {"fuse": "nvrtc"})
    assert ops_of(desc) == ["ChainerFusionGroup", "Relu"]
    assert "Mul Add Tanh Sigmoid Mul Add" in desc or sorted(lines(desc)[0].split(": ")[1].rstrip("]").split()) == \
        sorted("Mul Add Tanh Sigmoid Mul Add".split())
    # the hip set takes the whole chain; inputs in name order
    _, desc = vm.transform_onnx(m, {"fuse": "hip"})
    assert ops_of(desc) == ["ChainerFusionGroup"]
    assert lines(desc)[0].startswith("ChainerFusionGroup(a, b, c, x) -> (y)")
    # one calculation is not a group (min_fuse_ops = 2); Identity and Constant do not count
    m1 = model([("Add", ["x", "x"], ["t"]), ("Identity", ["t"], ["y"])], [("x", (3,))], [("y", (3,))])
    _, desc = vm.transform_onnx(m1, {"fuse": "hip"})
    assert ops_of(desc) == ["Add", "Identity"]


def test_fusion_rejects_cycles_and_unused_constants(vm):
    # s = Tanh(x); m = Softmax(s) (not fusable); y = Add(s, m): fusing Tanh and Add would put the
    # group both before and after Softmax
    m = model([("Tanh", ["x"], ["s"]), ("Softmax", ["s"], ["m"]), ("Add", ["s", "m"], ["y"])], [("x", (2, 3))], [("y", (2, 3))])
    _, desc = vm.transform_onnx(m, {"fuse": "hip"})
    assert ops_of(desc) == ["Tanh", "Softmax", "Add"]
    # with a second fusable node before the fork the front part still fuses
    m = model([("Exp", ["x"], ["e"]), ("Tanh", ["e"], ["s"]), ("Softmax", ["s"], ["m"]), ("Add", ["s", "m"], ["y"])],
              [("x", (2, 3))], [("y", (2, 3))])
    _, desc = vm.transform_onnx(m, {"fuse": "hip"})
    assert ops_of(desc) == ["ChainerFusionGroup", "Softmax", "Add"]
    # a one-element float constant joins the group that reads it; one that only outside nodes read does not
    k = onnx_lite.Node("Constant", [], ["k"], {"value": np.array(2.0, np.float32)})
    k2 = onnx_lite.Node("Constant", [], ["k2"], {"value": np.array(3.0, np.float32)})
    m = model([k, k2, ("Mul", ["x", "k"], ["t"]), ("Tanh", ["t"], ["u"]), ("Softmax", ["u"], ["v"]), ("Pow", ["v", "k2"], ["y"])],
              [("x", (2, 3))], [("y", (2, 3))])
    _, desc = vm.transform_onnx(m, {"fuse": "hip"})
    assert ops_of(desc) == ["Constant", "ChainerFusionGroup", "Softmax", "Pow"]
    assert "Constant Mul Tanh" in desc or "[hip #1: Constant Mul Tanh]" in desc


def test_groups_keep_to_one_result_shape(vm):
    # ReduceMax over everything gives a 0-d value; its product with a [6] constant has six elements.
    # One kernel writes every output of a group in the broadcast shape, so the two do not share a group.
    k = onnx_lite.Node("Constant", [], ["half"], {"value": np.array(0.5, np.float32)})
    w = onnx_lite.Node("Constant", [], ["w"], {"value": np.arange(6, dtype=np.float32)})
    red = onnx_lite.Node("ReduceMax", ["x"], ["m"], {"keepdims": 0})
    m = model([k, w, red, ("Mul", ["m", "half"], ["s"]), ("Abs", ["s"], ["t"]), ("Mul", ["t", "w"], ["u"]), ("Neg", ["u"], ["y"])],
              [("x", (4, 8))], [("y", (6,)), ("t", ())])
    _, desc = vm.transform_onnx(m, {"fuse": "hip"})
    groups = [l for l in lines(desc) if l.startswith("ChainerFusionGroup")]
    assert len(groups) == 2
    assert any("Mul Abs" in g and "-> (t)" in g for g in groups)
    assert any("Mul Neg" in g and "-> (y)" in g for g in groups)
    # operands of one shape: the chain stays whole
    m = model([("Mul", ["a", "b"], ["s"]), ("Abs", ["s"], ["t"]), ("Mul", ["t", "c"], ["u"]), ("Neg", ["u"], ["y"])],
              [("a", (4,)), ("b", (4,)), ("c", (4,))], [("y", (4,))])
    _, desc = vm.transform_onnx(m, {"fuse": "hip"})
    assert ops_of(desc) == ["ChainerFusionGroup"]


def test_dynamic_quantize_linear_is_expanded(vm):
    """DynamicQuantizeLinear becomes the body of its ONNX function (compiler/simplifier.cc:825-888 with
    the schema of ONNX 1.5): same node types, in that order, and the three outputs keep their names."""
    g = onnx_lite.Graph()
    g.name = "dql"
    g.nodes = [onnx_lite.Node("DynamicQuantizeLinear", ["x"], ["y", "s", "z"])]
    g.inputs = [("x", F, [3, 4])]
    g.outputs = [("y", onnx_lite.ONNX_OF[np.dtype(np.uint8)], [3, 4]), ("s", F, []), ("z", onnx_lite.ONNX_OF[np.dtype(np.uint8)], [])]
    _, desc = vm.transform_onnx(onnx_lite.make_model(g), {"fuse": "none"})
    assert sorted(ops_of(desc)) == sorted(["Constant", "Constant", "ReduceMin", "Min", "ReduceMax", "Max", "Sub", "Div", "Div", "Sub",
                                           "Clip", "Round", "Cast", "Identity", "Identity", "QuantizeLinear"])
    by_out = {l.split("-> (")[1].split(")")[0]: l for l in lines(desc)}
    assert by_out["y"].startswith("QuantizeLinear(x, ") and by_out["s"].startswith("Identity(") and by_out["z"].startswith("Identity(")
    # with the hip rule the 0-d arithmetic between the reductions and the Cast is one group
    _, desc = vm.transform_onnx(onnx_lite.make_model(g), {"fuse": "hip"})
    groups = [l for l in lines(desc) if l.startswith("ChainerFusionGroup")]
    assert len(groups) == 1 and "Clip" in groups[0] and "Round" in groups[0]
    insts = decode_program(vm, vm.compile_onnx(onnx_lite.make_model(g), {"fuse": "none"}))
    names = [i[0] for i in insts]
    assert "Clip" in names and "Round" in names and names.count("Out") == 3


def test_hip_program_text_compiles(vm):
    capi = pkg.capi
    k = onnx_lite.Node("Constant", [], ["half"], {"value": np.array(0.5, np.float32)})
    clip = onnx_lite.Node("Clip", ["t1"], ["t2"], {"min": 0.0, "max": 6.0})
    m = model([k, ("Mul", ["x", "half"], ["t0"]), ("Add", ["t0", "b"], ["t1"]), clip, ("Neg", ["t2"], ["y"])],
              [("x", (4, 8)), ("b", (8,))], [("y", (4, 8))])
    text = vm.fusion_program(m, 1, {"fuse": "hip"})
    st = [l for l in text.splitlines()]
    assert st[0] == "chxhip-fusion 1" and st[1] == "in v_fi000_b:float32 v_fi001_x:float32"
    assert st[2].endswith("= Const 0x3f000000")
    assert [l.split(" = ")[1].split()[0] for l in st[2:-1]] == ["Const", "Mul", "Add", "Clip", "Neg"]
    assert "0x00000000 0x40c00000" in st[5] and st[-1].startswith("out ") and st[-1].endswith(":float32")
    # the generator accepts it and hiprtc compiles the kernel for gfx950 (host only)
    full = capi.make_desc(0x10000000, capi.FLOAT32, (4, 8), (32, 4))
    vec = capi.make_desc(0x20000000, capi.FLOAT32, (8,), (4,))
    src = capi.elementwise_source(text, 1, [vec, full], [full], compile=True)
    assert "fusion1_" in src


def test_quantize_dequantize_parameters_are_written_into_the_group(vm):
    """QuantizeLinear / DequantizeLinear with constant parameters fuse (hip set only); the scale and
    zero point are no operands of the kernel."""
    inits = {"s1": np.array(0.05, np.float32), "z1": np.array(128, np.uint8), "s2": np.array(0.02, np.float32),
             "z2": np.array(3, np.int8), "s3": np.array(0.06, np.float32), "z3": np.array(7, np.uint8)}
    g = onnx_lite.Graph()
    g.nodes = [onnx_lite.Node("DequantizeLinear", ["a", "s1", "z1"], ["fa"]), onnx_lite.Node("DequantizeLinear", ["b", "s2", "z2"], ["fb"]),
               onnx_lite.Node("Add", ["fa", "fb"], ["s"]), onnx_lite.Node("Relu", ["s"], ["r"]),
               onnx_lite.Node("QuantizeLinear", ["r", "s3", "z3"], ["q"])]
    g.inputs = [("a", onnx_lite.UINT8, [2, 16, 4, 4]), ("b", onnx_lite.INT8, [2, 16, 4, 4])]
    g.inputs += [(k, onnx_lite.ONNX_OF[v.dtype], []) for k, v in inits.items()]
    g.outputs = [("q", onnx_lite.UINT8, [2, 16, 4, 4])]
    g.initializers = inits
    m = onnx_lite.make_model(g)
    _, desc = vm.transform_onnx(m, {"fuse": "nvrtc"})
    assert ops_of(desc) == ["DequantizeLinear", "DequantizeLinear", "Add", "Relu", "QuantizeLinear"]   # Add alone is no group
    text = vm.fusion_program(m, 1, {"fuse": "hip"})
    st = text.splitlines()
    assert st[1].split()[1:] == ["v_fi000_a:uint8", "v_fi001_b:int8"]
    assert "DequantizeLinear v_fi000_a 0x3d4ccccd 128" in text and "DequantizeLinear v_fi001_b 0x3ca3d70a 3" in text
    assert st[-2].endswith("0x3d75c28f 7 uint8") and st[-1].endswith(":uint8")
    # this is exactly the residual-sum group a convolution can absorb
    got = pkg.capi.match_residual_add(text)
    assert got is not None and got["relu"] and got["in_zero_point"] == [128, 3] and got["out_zero_point"] == 7
    # and the emitted instruction takes only the two tensors
    prog = vm.compile_onnx(m, {"fuse": "hip"})
    insts = decode_program(vm, prog)
    assert [i[0] for i in insts] == ["In", "In", "ElementWiseNvrtc", "Free", "Free", "Out"]
    assert insts[2][1][0] == ("ARRAY_LIST", [1, 2])


def decode_program(vm, data):
    """[(op name, [(value type name, value)], outputs)] of a serialized program."""
    return vm.decode_program(data)


def numpy_quantize(data, dtype):
    """compiler/quantize.cc:68-89, spelled with numpy float32 operations."""
    d = np.asarray(data, np.float32)
    rmin, rmax = np.float32(min(d.min(), 0)), np.float32(max(d.max(), 0))
    if dtype == np.int8:
        scale = np.float32(np.float32(max(abs(rmin), abs(rmax)) * np.float32(2)) / np.float32(254))
        return np.rint((d / scale).astype(np.float64)).astype(np.float32).astype(np.int8), scale, 0
    scale = np.float32((rmax - rmin) / np.float32(255)) if rmin != rmax else np.float32(1)
    zp = int(np.rint(np.float32(np.float32(0) - rmin) / scale))
    return (np.rint((d / scale).astype(np.float64)).astype(np.float32) + np.float32(zp)).astype(np.uint8), scale, zp


@pytest.mark.parametrize("dtype", [np.uint8, np.int8])
def test_weight_quantization_formulas(vm, dtype):
    rng = np.random.default_rng(5)
    for case in range(6):
        w = (rng.standard_normal((7, 5, 3)) * (0.01 + case)).astype(np.float32)
        if case == 1:
            w = np.abs(w)            # all positive: the range is widened to contain 0
        if case == 2:
            w = -np.abs(w)
        codes, scale, zp = vm.quantize_data(w, dtype)
        want, wscale, wzp = numpy_quantize(w, dtype)
        assert scale == wscale and zp == wzp
        np.testing.assert_array_equal(codes, want)
        # reconstruction error within half a step (one step at the clamped end of uint8)
        recon = (codes.astype(np.float32) - zp) * scale
        assert np.abs(recon - w).max() <= scale * 0.5001 + 1e-7
    codes, scale, zp = vm.quantize_data(np.zeros(4, np.float32), np.uint8)
    assert scale == 1 and zp == 0 and not codes.any()


CONV_ATTRS = {"strides": [2, 2], "pads": [1, 1, 1, 1], "kernel_shape": [3, 3], "group": 1, "dilations": [1, 1]}


def conv_model(rng, with_bias=False):
    w = (rng.standard_normal((6, 4, 3, 3)) * 0.2).astype(np.float32)
    inits = {"w": w}
    ins = ["x", "w"]
    if with_bias:
        inits["bias"] = np.zeros(6, np.float32)
        ins.append("bias")
    m = model([onnx_lite.Node("Conv", ins, ["y"], dict(CONV_ATTRS))], [("x", (1, 4, 8, 8))], [("y", (1, 6, 4, 4))], inits)
    return m, w


def test_quantizer_static_qlinear_rewrite(vm):
    rng = np.random.default_rng(6)
    m, w = conv_model(rng)
    opts = {"fuse": "none", "quantize": {"mode": "QLinearOps", "static": True, "asymmetric_input_types": True, "per_channel": True,
                                         "inputs": {"x": {"scale": 0.02, "zero_point": 121}},
                                         "outputs": {"y": {"scale": 0.05, "zero_point": 7, "dtype": "uint8"}}}}
    out, desc = vm.transform_onnx(m, opts)
    g = onnx_lite.parse_model(out)
    kinds = [n.op_type for n in g.nodes]
    assert sorted(kinds) == sorted(["Constant"] * 7 + ["QuantizeLinear", "QLinearConv", "DequantizeLinear"])
    const = {n.outputs[0]: n.attrs["value"] for n in g.nodes if n.op_type == "Constant"}
    q = next(n for n in g.nodes if n.op_type == "QuantizeLinear")
    conv = next(n for n in g.nodes if n.op_type == "QLinearConv")
    dq = next(n for n in g.nodes if n.op_type == "DequantizeLinear")
    # x -> QuantizeLinear(x, 0.02, uint8 121) -> QLinearConv(..) -> DequantizeLinear(.., 0.05, 7) -> y
    assert q.inputs[0] == "x" and const[q.inputs[1]] == np.float32(0.02) and const[q.inputs[2]] == 121 and const[q.inputs[2]].dtype == np.uint8
    assert conv.inputs[0] == q.outputs[0] and conv.inputs[1:3] == q.inputs[1:3]
    assert dq.inputs[0] == conv.outputs[0] and dq.outputs == ["y"] and dq.inputs[1:] == conv.inputs[6:8]
    assert const[conv.inputs[6]] == np.float32(0.05) and const[conv.inputs[7]] == 7
    for k, v in CONV_ATTRS.items():
        assert conv.attrs[k] == v
    # per-channel int8 weights: every output channel on its own scale
    wq, ws, wz = const[conv.inputs[3]], const[conv.inputs[4]], const[conv.inputs[5]]
    assert wq.dtype == np.int8 and wq.shape == w.shape and ws.shape == (6,) and wz.shape == (6,) and wz.dtype == np.int8 and not wz.any()
    for c in range(6):
        want, scale, _ = numpy_quantize(w[c], np.int8)
        np.testing.assert_array_equal(wq[c], want)
        assert ws[c] == scale
    # per tensor, uint8 weights (the reference's default input types)
    opts["quantize"].update(per_channel=False, asymmetric_input_types=False)
    g = onnx_lite.parse_model(vm.transform_onnx(m, opts)[0])
    const = {n.outputs[0]: n.attrs["value"] for n in g.nodes if n.op_type == "Constant"}
    conv = next(n for n in g.nodes if n.op_type == "QLinearConv")
    want, scale, zp = numpy_quantize(w, np.uint8)
    np.testing.assert_array_equal(const[conv.inputs[3]], want)
    assert const[conv.inputs[4]].shape == () and const[conv.inputs[4]] == scale and const[conv.inputs[5]] == zp
    # missing parameters are an error that names the value
    bad = {"fuse": "none", "quantize": {"mode": "QLinearOps", "static": True, "inputs": {"x": {"scale": 0.02, "zero_point": 1}}}}
    with pytest.raises(vm.ChxVMError, match="output 'y'"):
        vm.transform_onnx(m, bad)


def test_quantizer_dynamic_integer_rewrite(vm):
    """The default mode (compiler/passes.cc:121-125): parameters computed at run time, integer
    contraction, scale back in float."""
    rng = np.random.default_rng(7)
    m, w = conv_model(rng)
    out, desc = vm.transform_onnx(m, {"fuse": "none", "quantize": {"per_channel": True}})
    g = onnx_lite.parse_model(out)
    kinds = [n.op_type for n in g.nodes]
    for op, count in (("ReduceMin", 1), ("ReduceMax", 1), ("Sub", 2), ("Div", 2), ("Floor", 1), ("Cast", 2), ("QuantizeLinear", 1),
                      ("ConvInteger", 1), ("Mul", 2), ("Reshape", 1)):
        assert kinds.count(op) == count, (op, kinds)
    conv = next(n for n in g.nodes if n.op_type == "ConvInteger")
    for k, v in CONV_ATTRS.items():
        assert conv.attrs[k] == v
    const = {n.outputs[0]: n.attrs["value"] for n in g.nodes if n.op_type == "Constant"}
    want, scale, zp = numpy_quantize(w[0], np.uint8)
    np.testing.assert_array_equal(const[conv.inputs[1]][0], want)            # uint8 weights per channel
    reshape = next(n for n in g.nodes if n.op_type == "Reshape")
    assert const[reshape.inputs[1]].tolist() == [6, 1, 1]
    last = g.nodes[-1]
    assert last.op_type == "Mul" and last.outputs == ["y"]
    casts = [n for n in g.nodes if n.op_type == "Cast"]
    assert sorted(c.attrs["to"] for c in casts) == [onnx_lite.FLOAT, onnx_lite.UINT8]
    # int8 activations would use the symmetric formula; MatMul takes the same route, per tensor
    mm = model([("MatMul", ["a", "b"], ["y"])], [("a", (3, 5))], [("y", (3, 2))], {"b": rng.standard_normal((5, 2)).astype(np.float32)})
    g = onnx_lite.parse_model(vm.transform_onnx(mm, {"fuse": "none", "quantize": {}})[0])
    assert [n.op_type for n in g.nodes].count("MatMulInteger") == 1 and "Reshape" not in [n.op_type for n in g.nodes]
    # a convolution with a bias is left alone (compiler/quantize.cc:383-387)
    mb, _ = conv_model(rng, with_bias=True)
    g = onnx_lite.parse_model(vm.transform_onnx(mb, {"fuse": "none", "quantize": {}})[0])
    assert [n.op_type for n in g.nodes] == ["Conv"]


def test_emitted_program_for_a_quantized_convolution(vm):
    rng = np.random.default_rng(8)
    m, w = conv_model(rng)
    opts = {"quantize": {"mode": "QLinearOps", "static": True, "asymmetric_input_types": True, "per_channel": True,
                         "inputs": {"x": {"scale": 0.02, "zero_point": 121}}, "outputs": {"y": {"scale": 0.05, "zero_point": 7}}}}
    insts = decode_program(vm, vm.compile_onnx(m, opts))
    names = [i[0] for i in insts]
    assert names[0] == "In" and names[-1] == "Out"
    assert names.count("QuantizeLinear") == 1 and names.count("QLinearConv") == 1 and names.count("DequantizeLinear") == 1
    conv = next(i for i in insts if i[0] == "QLinearConv")
    kinds = [t for t, _ in conv[1]]
    assert kinds == ["ARRAY", "SCALAR", "SCALAR", "ARRAY", "ARRAY", "ARRAY", "SCALAR", "SCALAR", "ARRAY", "INTS", "INTS", "INT", "STRING"]
    assert conv[1][8][1] == -1 and conv[1][9][1] == [2, 2] and conv[1][10][1] == [1, 1] and conv[1][11][1] == 1 and conv[1][12][1] == ""
    # scales and zero points of the activations are scalar constants, the per-channel weight parameters arrays
    assert names.count("FloatScalarConstant") == 2 and names.count("IntScalarConstant") == 2
    assert names.count("IntConstant") == 2 and names.count("FloatConstant") == 1
    # every temporary is freed after its last reader; the program survives the C++ reader and writer
    assert names.count("Free") >= 3
    data = vm.compile_onnx(m, opts)
    assert vm.proto_roundtrip(data) == data
    # node types outside the path are refused by the emitter, by name
    sm = model([("LogSoftmax", ["x"], ["y"])], [("x", (2, 3))], [("y", (2, 3))])
    with pytest.raises(vm.ChxVMError, match="LogSoftmax"):
        vm.compile_onnx(sm)
    with pytest.raises(vm.ChxVMError, match="unknown option"):
        vm.compile_onnx(sm, {"fuze": "hip"})


def test_reference_flag_names_as_options(vm):
    """The compiler flags of the reference that concern this path are accepted under their own names
    (scripts/generate_flags_code.py:4-173; use_hip beside use_nvrtc): quantize as a bool selects the
    default mode with per-channel weights (compiler/passes.cc:121-125, compiler/quantize.h:34),
    disable_per_channel_quantize clears that; fuse_operations + use_hip / use_nvrtc choose the groups."""
    rng = np.random.default_rng(9)
    m, w = conv_model(rng)

    def kinds(options):
        return [n.op_type for n in onnx_lite.parse_model(vm.transform_onnx(m, options)[0]).nodes]
    per_channel = kinds({"fuse_operations": False, "quantize": True})
    assert per_channel == kinds({"fuse": "none", "quantize": {"per_channel": True}}) == kinds({"fuse": "none", "quantize": {}})
    assert "Reshape" in per_channel and "ConvInteger" in per_channel               # [OC] scales reshaped to [OC, 1, 1]
    per_tensor = kinds({"fuse_operations": False, "quantize": True, "disable_per_channel_quantize": True})
    assert per_tensor == kinds({"fuse": "none", "quantize": {"per_channel": False}}) and "Reshape" not in per_tensor
    assert kinds({"quantize": False, "fuse_operations": False}) == ["Conv"]
    chain = model([("Tanh", ["x"], ["t"]), ("Sigmoid", ["t"], ["s"]), ("Relu", ["s"], ["y"])], [("x", (4, 5))], [("y", (4, 5))])

    def groups(options):
        return lines(vm.transform_onnx(chain, options)[1])
    assert groups({"fuse_operations": True, "use_hip": True, "backend_name": "hip"}) == groups({"fuse": "hip"})
    assert groups({"fuse_operations": True, "use_nvrtc": True}) == groups({"fuse": "nvrtc"})
    assert groups({"fuse_operations": False, "use_hip": True}) == groups({"fuse": "none"})
    assert [l.split("(")[0] for l in groups({"fuse": "none"})] == ["Tanh", "Sigmoid", "Relu"]
    assert groups({"fuse": "hip"}) != groups({"fuse": "nvrtc"})                     # Relu is fusable for hip only
    with pytest.raises(vm.ChxVMError, match="backend_name"):
        vm.transform_onnx(chain, {"backend_name": "chxvm"})
    with pytest.raises(vm.ChxVMError, match="unknown option 'use_tvm'"):
        vm.transform_onnx(chain, {"use_tvm": True})


def test_float_head_nodes_are_emitted_with_the_reference_operand_lists(vm):
    """Flatten, Gemm, MatMul (compiler/chxvm/simple_node_emitter.cc:312-318, 698-701): operands in the order of
    runtime/chxvm_defs.py, attribute defaults of the ONNX nodes (alpha = beta = 1, no transposition, axis 1)."""
    N = onnx_lite.Node
    w, b, w2 = np.zeros((9, 32), np.float32), np.zeros(9, np.float32), np.zeros((9, 4), np.float32)
    m = model([N("Flatten", ["x"], ["f"], {}), N("Gemm", ["f", "w", "b"], ["h"], {"transB": 1, "alpha": 0.5}), N("Gemm", ["h", "w2"], ["h2"], {}),
               N("MatMul", ["h2", "w3"], ["y"], {})],
              [("x", (3, 2, 4, 4))], [("y", (3, 4))], {"w": w, "b": b, "w2": w2, "w3": np.zeros((4, 4), np.float32)})
    insts = decode_program(vm, vm.compile_onnx(m, {"fuse": "none"}))
    flat = next(i for i in insts if i[0] == "Flatten")
    assert [t for t, _ in flat[1]] == ["ARRAY", "INT"] and flat[1][1][1] == 1
    g1, g2 = [i for i in insts if i[0] == "Gemm"]
    assert [t for t, _ in g1[1]] == ["ARRAY", "ARRAY", "ARRAY", "FLOAT", "FLOAT", "INT", "INT"]
    assert [v for _, v in g1[1][3:]] == [0.5, 1.0, 0, 1] and g1[1][2][1] > 0
    assert [v for _, v in g2[1][2:]] == [-1, 1.0, 1.0, 0, 0]          # no c: the optional operand is -1
    mm = next(i for i in insts if i[0] == "MatMul")
    assert [t for t, _ in mm[1]] == ["ARRAY", "ARRAY"]


def test_global_pools_become_pools_over_the_spatial_extent(vm):
    """ReplaceGlobalPool, compiler/simplifier.cc:272-290: kernel_shape = the input's spatial dimensions, which have to
    be known; strides 1 and no padding are the pool nodes' defaults."""
    N = onnx_lite.Node
    m = model([N("GlobalAveragePool", ["x"], ["a"], {}), N("GlobalMaxPool", ["x"], ["y"], {})], [("x", (2, 8, 7, 5))],
              [("a", (2, 8, 1, 1)), ("y", (2, 8, 1, 1))])
    insts = decode_program(vm, vm.compile_onnx(m, {"fuse": "none"}))
    avg = next(i for i in insts if i[0] == "AveragePool")
    assert [t for t, _ in avg[1]] == ["ARRAY", "INTS", "INTS", "INTS", "INT"]
    assert [list(v) if isinstance(v, (list, tuple)) else v for _, v in avg[1][1:]] == [[7, 5], [1, 1], [0, 0], 0]
    mx = next(i for i in insts if i[0] == "MaxPool")
    assert [list(v) if isinstance(v, (list, tuple)) else v for _, v in mx[1][1:]] == [[7, 5], [1, 1], [0, 0], 0, "NOTSET"]
    assert avg[2][1] == -1 and mx[2][1] == -1          # the backward context is dropped
    unknown = model([N("MaxPool", ["x"], ["h"], {"kernel_shape": [2, 2]}), N("GlobalAveragePool", ["h"], ["a"], {})], [("x", (2, 8, 7, 5))], [("a", (2, 8, 1, 1))])
    with pytest.raises(vm.ChxVMError, match="shape of GlobalAveragePool must be known"):
        vm.compile_onnx(unknown, {"fuse": "none"})


def test_batch_normalization_is_emitted_in_its_inference_form(vm):
    """EmitBatchNormalization, compiler/chxvm/emitter.cc:193-206: one output -> FixedBatchNormalization(x, s, bias, mean, var,
    epsilon); the outputs of a training step are not on this path."""
    N = onnx_lite.Node
    c4 = {k: np.ones(4, np.float32) for k in ("s", "b", "m", "v")}
    m = model([N("BatchNormalization", ["x", "s", "b", "m", "v"], ["y"], {"epsilon": 1e-3})], [("x", (2, 4, 3, 3))], [("y", (2, 4, 3, 3))], c4)
    insts = decode_program(vm, vm.compile_onnx(m, {"fuse": "none"}))
    bn = next(i for i in insts if i[0] == "FixedBatchNormalization")
    assert [t for t, _ in bn[1]] == ["ARRAY"] * 5 + ["FLOAT"] and abs(bn[1][5][1] - 1e-3) < 1e-9
    assert not any(i[0] == "BatchNormalization" for i in insts)
    train = model([N("BatchNormalization", ["x", "s", "b", "m", "v"], ["y", "rm", "rv"], {})], [("x", (2, 4, 3, 3))],
                  [("y", (2, 4, 3, 3)), ("rm", (4,)), ("rv", (4,))], c4)
    with pytest.raises(vm.ChxVMError, match=r"1 vs\. 3.*BatchNormalization"):
        vm.compile_onnx(train, {"fuse": "none"})


def test_float_conv_is_emitted_with_the_reference_operand_list(vm):
    """compiler/chxvm/simple_node_emitter.cc:213-219: Conv(x, w, b?, strides, pads, group, auto_pad); the quantizer leaves
    a Conv with a bias as it is (compiler/quantize.cc:376-381) and rewrites the one without."""
    rng = np.random.default_rng(9)
    m, _ = conv_model(rng, with_bias=True)
    insts = decode_program(vm, vm.compile_onnx(m, {"quantize": {}}))
    conv = next(i for i in insts if i[0] == "Conv")
    assert [t for t, _ in conv[1]] == ["ARRAY", "ARRAY", "ARRAY", "INTS", "INTS", "INT", "STRING"]
    assert not any(i[0] == "ConvInteger" for i in insts)
    m, _ = conv_model(rng, with_bias=False)
    insts = decode_program(vm, vm.compile_onnx(m, {"fuse": "none"}))                     # not quantized at all: a float Conv, no bias
    conv = next(i for i in insts if i[0] == "Conv")
    assert conv[1][2][1] == -1


def test_view_nodes_are_emitted_with_the_reference_operand_lists(vm):
    """Transpose(data, perm), Squeeze(data, axes), Unsqueeze(data, sorted axes): compiler/chxvm/simple_node_emitter.cc:297-311,
    523-526; Unsqueeze refuses negative and positive axes together."""
    N = onnx_lite.Node
    m = model([N("Transpose", ["x"], ["t"], {"perm": [1, 0, 2]}), N("Squeeze", ["t"], ["s"], {"axes": [2]}), N("Unsqueeze", ["s"], ["y"], {"axes": [3, 0]})],
              [("x", (2, 3, 1))], [("y", (1, 3, 2, 1))])
    insts = {i[0]: i for i in decode_program(vm, vm.compile_onnx(m, {"fuse": "none"}))}
    assert list(insts["Transpose"][1][1][1]) == [1, 0, 2] and list(insts["Squeeze"][1][1][1]) == [2]
    assert list(insts["Unsqueeze"][1][1][1]) == [0, 3]
    mixed = model([N("Unsqueeze", ["x"], ["y"], {"axes": [-1, 1]})], [("x", (2, 3))], [("y", (2, 1, 3, 1))])
    with pytest.raises(vm.ChxVMError, match="mixed"):
        vm.compile_onnx(mixed, {"fuse": "none"})


def test_concat_is_emitted_with_an_array_list(vm):
    """compiler/chxvm/simple_node_emitter.cc:490-494: Concat(inputs as one list, axis)."""
    N = onnx_lite.Node
    m = model([N("Concat", ["a", "b", "a"], ["y"], {"axis": 2})], [("a", (2, 3, 1)), ("b", (2, 3, 4))], [("y", (2, 3, 6))])
    cat = next(i for i in decode_program(vm, vm.compile_onnx(m, {"fuse": "none"})) if i[0] == "Concat")
    assert [t for t, _ in cat[1]] == ["ARRAY_LIST", "INT"] and len(cat[1][0][1]) == 3 and cat[1][1][1] == 2
