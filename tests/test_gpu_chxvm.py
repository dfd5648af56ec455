"""Serialized ChxVM programs run by the C++ VM of the hip runtime (proto reader -> generated op
classes -> RunImpl bodies -> C ABI), compared with the CPU oracle: bit-exact for the 8-bit and
int32 results, and for the fused fp32 chain (the device code restates the host libm bit for bit;
the stated bar is 2 ulp or 1e-6 relative)."""
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


def rand_q(rng, shape, dtype):
    lo, hi = (0, 256) if dtype == np.uint8 else (-128, 128)
    return rng.integers(lo, hi, size=shape).astype(dtype)


def test_quantize_dequantize_program(g, vm, oracle):
    b = vm.ProgramBuilder()
    x = b.input("x", "float32", (3, 5, 7))
    s = b.scalar(0.037, "float32")
    z = b.scalar(131, "uint8")
    q = b.QuantizeLinear(x, s, z)
    d = b.DequantizeLinear(q, s, z)
    q0 = b.QuantizeLinear(x, s, None)          # absent zero point: uint8 0
    b.output("q", q)
    b.output("d", d)
    b.output("q0", q0)
    prog = vm.Program(b.serialize())
    assert prog.num_instructions == 9 and prog.input_names == ["x"]
    rng = np.random.default_rng(3)
    xv = (rng.standard_normal((3, 5, 7)) * 3).astype(np.float32)
    out = prog.run({"x": g.dev(xv)})
    want_q = oracle.quantize_linear(xv, np.float32(0.037), 131, np.uint8)
    np.testing.assert_array_equal(out["q"], want_q)
    np.testing.assert_array_equal(out["d"].view(np.int32), oracle.dequantize_linear(want_q, np.float32(0.037), 131).view(np.int32))
    np.testing.assert_array_equal(out["q0"], oracle.quantize_linear(xv, np.float32(0.037), 0, np.uint8))
    assert out["q"].dtype == np.uint8 and out["d"].dtype == np.float32
    # a second run of the same program object gives the same values
    np.testing.assert_array_equal(prog.run({"x": g.dev(xv)})["q"], want_q)


def test_int8_zero_point_selects_int8_output(g, vm, oracle):
    b = vm.ProgramBuilder()
    x = b.input("x")
    q = b.QuantizeLinear(x, b.scalar(0.5, "float32"), b.scalar(-7, "int8"))
    b.output("q", q)
    xv = np.linspace(-80, 80, 1001).astype(np.float32)
    out = vm.Program(b.serialize()).run({"x": g.dev(xv)})
    assert out["q"].dtype == np.int8
    np.testing.assert_array_equal(out["q"], oracle.quantize_linear(xv, np.float32(0.5), -7, np.int8))


@pytest.mark.parametrize("auto_pad,pads,strides", [("", [1, 1], [1, 1]), ("SAME_UPPER", [], [2, 2]), ("", [], [])])
def test_qlinear_conv_program(g, vm, oracle, auto_pad, pads, strides):
    """In -> QuantizeLinear -> QLinearConv (constants as instructions, bias added the reference's
    way) -> DequantizeLinear -> Out, twice through the same program (the plan is built once)."""
    rng = np.random.default_rng(11)
    N, C, H, W, OC = 2, 16, 9, 10, 24
    w = rng.integers(-127, 128, size=(OC, C, 3, 3)).astype(np.int8)
    ws = rng.uniform(0.001, 0.01, size=OC).astype(np.float32)
    wz = np.zeros(OC, np.int8)
    bias = rng.integers(-5, 6, size=OC).astype(np.int32)
    xs, xz, ys, yz = np.float32(0.02), 128, np.float32(0.11), 120
    b = vm.ProgramBuilder()
    x = b.input("x", "float32", (N, C, H, W))
    s_x, z_x = b.scalar(float(xs), "float32"), b.scalar(xz, "uint8")
    q = b.QuantizeLinear(x, s_x, z_x)
    y = b.QLinearConv(q, s_x, z_x, b.constant(w), b.constant(ws), b.constant(wz), b.scalar(float(ys), "float32"),
                      b.scalar(yz, "uint8"), b.constant(bias), strides, pads, 1, auto_pad)
    d = b.DequantizeLinear(y, b.scalar(float(ys), "float32"), b.scalar(yz, "uint8"))
    b.Free(q)
    b.output("y", y)
    b.output("d", d)
    prog = vm.Program(b.serialize())
    for seed in (0, 1):
        xv = np.random.default_rng(seed).uniform(-2.5, 2.5, size=(N, C, H, W)).astype(np.float32)
        out = prog.run({"x": g.dev(xv)})
        qx = oracle.quantize_linear(xv, xs, xz, np.uint8)
        want = oracle.qlinear_conv_int(qx, xs, xz, w, ws, wz, ys, yz, np.uint8, bias=bias,
                                       bias_mode=oracle.BIAS_REFERENCE_FLOAT, strides=tuple(strides) or (1, 1),
                                       pads=tuple(pads) or (0, 0), auto_pad=auto_pad)
        np.testing.assert_array_equal(out["y"], want)
        assert want.min() < want.max()
        np.testing.assert_array_equal(out["d"].view(np.int32), oracle.dequantize_linear(want, ys, yz).view(np.int32))


def test_qlinear_conv_onnx_vector_through_vm(g, vm, onnx_vectors):
    t = onnx_vectors["test_qlinearconv"]
    b = vm.ProgramBuilder()
    x = b.input("x", "uint8", t["x_shape"])
    y = b.QLinearConv(x, b.scalar(t["x_scale"], "float32"), b.scalar(t["x_zero_point"], "uint8"),
                      b.constant(np.array(t["w"], np.uint8).reshape(t["w_shape"])),
                      b.constant(np.array(t["w_scale"], np.float32)), b.constant(np.array(t["w_zero_point"], np.uint8)),
                      b.scalar(t["y_scale"], "float32"), b.scalar(t["y_zero_point"], "uint8"), None, [], [], 1, "")
    b.output("y", y)
    out = vm.Program(b.serialize()).run({"x": g.dev(np.array(t["x"], np.uint8).reshape(t["x_shape"]))})
    assert out["y"].reshape(7, 7).tolist() == t["y"]


def test_conv_integer_and_matmul_integer_programs(g, vm, oracle, onnx_vectors):
    rng = np.random.default_rng(5)
    x, w = rand_q(rng, (2, 6, 9, 8), np.uint8), rand_q(rng, (4, 3, 3, 2), np.int8)
    wz = rand_q(rng, (4,), np.int8)
    b = vm.ProgramBuilder()
    xi = b.input("x", "uint8", x.shape)
    y = b.ConvInteger(xi, b.constant(w), b.scalar(77, "uint8"), b.constant(wz), [2, 1], [0, 1], 2, "")
    y2 = b.ConvInteger(xi, b.constant(w), None, None, [2, 1], [0, 1], 2, "")
    b.output("y", y)
    b.output("y2", y2)
    out = vm.Program(b.serialize()).run({"x": g.dev(x)})
    np.testing.assert_array_equal(out["y"], oracle.conv_integer(x, w, 77, wz, strides=(2, 1), pads=(0, 1), group=2))
    np.testing.assert_array_equal(out["y2"], oracle.conv_integer(x, w, None, None, strides=(2, 1), pads=(0, 1), group=2))
    assert out["y"].dtype == np.int32

    t = onnx_vectors["test_matmulinteger"]
    b = vm.ProgramBuilder()
    a, bb = b.input("a", "uint8"), b.input("b", "uint8")
    y = b.MatMulInteger(a, bb, b.constant(np.array([t["a_zero_point"]], np.uint8)),
                        b.constant(np.array([t["b_zero_point"]], np.uint8)))
    b.output("y", y)
    out = vm.Program(b.serialize()).run({"a": g.dev(np.array(t["a"], np.uint8)), "b": g.dev(np.array(t["b"], np.uint8))})
    assert out["y"].tolist() == t["y"]
    a_, b_ = rand_q(rng, (3, 5, 37), np.uint8), rand_q(rng, (3, 37, 11), np.int8)
    b = vm.ProgramBuilder()
    y = b.MatMulInteger(b.input("a", "uint8"), b.input("b", "int8"), None, None)
    b.output("y", y)
    out = vm.Program(b.serialize()).run({"a": g.dev(a_), "b": g.dev(b_)})
    np.testing.assert_array_equal(out["y"], oracle.matmul_integer(a_, b_, None, None))


def test_fusion_group_program(g, vm, oracle):
    """ElementWiseNvrtc with the chain Mul, Add, Tanh, Sigmoid, Mul, Add, Relu and broadcast
    [C] operands; two outputs."""
    chain = [("t0", "Mul", "x", "a"), ("t1", "Add", "t0", "b"), ("t2", "Tanh", "t1"), ("t3", "Sigmoid", "t2"),
             ("t4", "Mul", "t3", "x"), ("t5", "Add", "t4", "c"), ("y", "Relu", "t5")]
    code = g.ops.fusion_program(
        [("x", torch.float32), ("a", torch.float32), ("b", torch.float32), ("c", torch.float32)], chain,
        [("y", torch.float32), ("t2", torch.float32)])
    b = vm.ProgramBuilder()
    ins = [b.input(n) for n in ("x", "a", "b", "c")]
    y, t2 = b.ElementWiseNvrtc(ins, 2, code, 3, num_list_outputs=2)
    b.output("y", y)
    b.output("t2", t2)
    prog = vm.Program(b.serialize())
    rng = np.random.default_rng(9)
    x = rng.standard_normal((4, 33, 65)).astype(np.float32) * 2
    a, bb = rng.standard_normal(65).astype(np.float32), rng.standard_normal(65).astype(np.float32)
    c = rng.standard_normal((4, 33, 65)).astype(np.float32)
    out = prog.run({"x": g.dev(x), "a": g.dev(a), "b": g.dev(bb), "c": g.dev(c)})
    env = oracle.run_chain(chain, {"x": x, "a": a, "b": bb, "c": c})
    t2w, yw = env["t2"], env["y"]
    # bar: 2 ulp or 1e-6 relative; the device code is written to give 0
    assert g.ulp_diff(out["t2"], t2w).max() == 0
    assert g.ulp_diff(out["y"], yw).max() == 0


def test_null_operand_skips_the_op(g, vm):
    """An op with a null array operand is skipped and its outputs become null
    (runtime/gen_chxvm.py:240-253); reading such an output as an array fails."""
    b = vm.ProgramBuilder()
    n = b.NullConstant()
    q = b.QuantizeLinear(n, b.scalar(1.0, "float32"), None)
    i = b.new_slot()
    b.add("Identity", q, outputs=[i])
    b.output("q", i)
    prog = vm.Program(b.serialize())
    with pytest.raises(vm.ChxVMError):
        prog.run({})


def test_errors_name_the_instruction(g, vm):
    b = vm.ProgramBuilder()
    x = b.input("x")
    b.output("y", b.QuantizeLinear(x, b.scalar(1.0, "float32"), b.scalar(3, "int32"), debug_info="node quant0"))
    prog = vm.Program(b.serialize())
    with pytest.raises(vm.ChxVMError) as e:
        prog.run({"x": g.dev(np.zeros(4, np.float32))})
    assert "uint8 or int8" in str(e.value)
    with pytest.raises(vm.ChxVMError) as e:
        prog.run({})
    assert "Input 'x' not found" in str(e.value)
    # writing a slot twice is refused (runtime/chxvm_state.cc:171-176)
    b = vm.ProgramBuilder()
    x = b.input("x")
    s = b.scalar(1.0, "float32")
    q = b.QuantizeLinear(x, s, None)
    b.add("QuantizeLinear", x, s, -1, outputs=[q])
    with pytest.raises(vm.ChxVMError):
        vm.Program(b.serialize()).run({"x": g.dev(np.zeros(4, np.float32))})


def _run_network_through_vm(g, vm, oracle, model, keep, fused_residuals=None, paired=None, minus_128=None):
    wl = g.pkg.workloads
    before = vm.counter("qlinearconv_residual_fusions")
    pairs_before = vm.counter("qlinearconv_pair_fusions")
    stores_before = vm.counter("minus_128_stores")
    serialized = wl.program_to_chxvm(model, vm, g.pkg.ops, keep=keep).serialize()
    assert vm.proto_roundtrip(serialized) == serialized
    vm.set_option("qlinearconv_bias", "onnx_int32")
    try:
        prog = vm.Program(serialized)
        got = prog.run({"x": torch.from_numpy(model["input"]).cuda()})
        prog.close()
    finally:
        vm.set_option("qlinearconv_bias", "reference")
    oracle.set_threads(16)
    try:
        ref = wl.run_reference(model, oracle, model["input"], keep=set(keep))
    finally:
        oracle.set_threads(1)
    assert sorted(got) == sorted(keep)
    for name in keep:
        np.testing.assert_array_equal(got[name], ref[name], err_msg="value %s" % name)
    if fused_residuals is not None:
        assert vm.counter("qlinearconv_residual_fusions") - before == fused_residuals
    if paired is not None:
        assert vm.counter("qlinearconv_pair_fusions") - pairs_before == paired
    if minus_128 is not None:
        assert vm.counter("minus_128_stores") - stores_before == minus_128


def test_small_resnet_as_one_program(g, vm, oracle):
    """The reduced ResNet as one serialized program: QuantizeLinear, QLinearConv with constant
    operands, DequantizeLinear -> MaxPool / AveragePool -> QuantizeLinear fused at load,
    FusionGroups for the residual sums, Free after the last reader.  Every value, then only the logits."""
    model = g.pkg.workloads.build_resnet50(batch=2, image=64, seed=5, width=16, blocks=(2, 1, 1, 1), classes=10)
    # The two convolutions that read a down-sampling block's input run as one launch where the first has a multiple of
    # 64 output channels (the blocks with 64 and 128 channels here; the other two pairs run one after the other).
    wl = g.pkg.workloads
    pairs = sum(1 for ins in wl.pair_convolutions(model["program"], model["convs"]) if ins[0] == "QLinearConvPair")
    assert pairs == 2
    # every value is a program output: nothing may be absorbed into another instruction
    # (a program output is read as plain codes: no value is kept as code - 128)
    _run_network_through_vm(g, vm, oracle, model, [ins[1] for ins in model["program"]], fused_residuals=0, paired=pairs, minus_128=0)
    # only the logits: each of the five residual sums is computed by the convolution before it
    blocks = sum(1 for ins in model["program"] if ins[0] == "AddRelu")
    assert blocks == 5
    # The values only convolutions read (as input or as the residual operand of an absorbed sum) are kept as
    # code - 128: what the Python runner's analysis finds on the same program with the same fusions.
    runner = wl.DeviceRunner(model, g.pkg, fuse_residual=True, pair_convs=True, minus_128=True)
    kept_minus_128 = len(runner.minus_128)
    runner.close()
    assert kept_minus_128 >= 8
    _run_network_through_vm(g, vm, oracle, model, ["logits"], fused_residuals=blocks, paired=pairs, minus_128=kept_minus_128)
    # the block outputs too: the sums are still absorbed (their convolutions' results are not outputs), and come out
    # as plain codes
    keep = ["logits"] + [ins[1] for ins in model["program"] if ins[0] == "AddRelu"]
    _run_network_through_vm(g, vm, oracle, model, keep, fused_residuals=blocks, paired=pairs)
    vm.set_option("store_minus_128", "off")
    try:
        _run_network_through_vm(g, vm, oracle, model, ["logits"], fused_residuals=blocks, paired=pairs, minus_128=0)
    finally:
        vm.set_option("store_minus_128", "on")
    # residual sums as instructions of their own: the operand a sum reads is then not one only convolutions read
    vm.set_option("fuse_residual", "off")
    vm.set_option("pair_convolutions", "off")
    try:
        _run_network_through_vm(g, vm, oracle, model, keep, fused_residuals=0, paired=0)
        _run_network_through_vm(g, vm, oracle, model, ["logits"], fused_residuals=0, paired=0)
    finally:
        vm.set_option("fuse_residual", "on")
        vm.set_option("pair_convolutions", "on")


def test_small_mobilenetv2_as_one_program(g, vm, oracle):
    """Depthwise convolutions and 24-channel activations (pixel pitch padded to 16 bytes) in the VM."""
    blocks = ((1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 1, 2))
    model = g.pkg.workloads.build_mobilenetv2(batch=2, image=64, seed=7, blocks=blocks, stem=32, head=128, classes=10)
    _run_network_through_vm(g, vm, oracle, model, [ins[1] for ins in model["program"]], fused_residuals=0)
    adds = [ins[1] for ins in model["program"] if ins[0] == "Add"]
    assert len(adds) >= 1
    _run_network_through_vm(g, vm, oracle, model, ["logits"] + adds, fused_residuals=len(adds))
    # only the logits: the block outputs and the depthwise results are kept as code - 128 between the convolutions, the
    # values the Python runner's analysis names on the same program (the expansion results, which a depthwise
    # convolution reads, keep plain codes)
    runner = g.pkg.workloads.DeviceRunner(model, g.pkg, fuse_residual=True, pair_convs=True, minus_128=True)
    kept_minus_128 = len(runner.minus_128)
    runner.close()
    depthwise = sum(1 for c in model["convs"].values() if c.group > 1)
    assert kept_minus_128 >= depthwise >= 3
    _run_network_through_vm(g, vm, oracle, model, ["logits"], fused_residuals=len(adds), minus_128=kept_minus_128)


def test_residual_group_with_other_constants_runs_unfused(g, vm, oracle):
    """A group whose DequantizeLinear constants are not the convolution's output quantization is not
    the convolution's to compute: both instructions run as they are, and the result is the oracle's."""
    rng = np.random.default_rng(77)
    x = rand_q(rng, (1, 16, 6, 6), np.uint8)
    w = rng.integers(-127, 128, size=(32, 16, 1, 1)).astype(np.int8)
    ws = rng.uniform(0.002, 0.02, size=32).astype(np.float32)
    r = rand_q(rng, (1, 32, 6, 6), np.uint8)
    u8 = torch.uint8

    def scale_bits(v):
        return "0x%08x" % np.float32(v).view(np.uint32)
    for group_scale, expect in ((0.25, 1), (0.26, 0)):
        code = g.ops.fusion_program(
            [("a", u8), ("b", u8)],
            [("fa", "DequantizeLinear", "a", scale_bits(group_scale), 120), ("fb", "DequantizeLinear", "b", scale_bits(0.1), 3),
             ("s", "Add", "fb", "fa"), ("q", "QuantizeLinear", "s", scale_bits(0.3), 100, "uint8")], [("q", u8)])
        b = vm.ProgramBuilder()
        xs = b.input("x", "uint8", x.shape)
        rs = b.input("r", "uint8", r.shape)
        y = b.QLinearConv(xs, b.scalar(0.02, "float32"), b.scalar(128, "uint8"), b.constant(w), b.constant(ws),
                          b.constant(np.zeros(32, np.int8)), b.scalar(0.25, "float32"), b.scalar(120, "uint8"), None, [1, 1], [0, 0], 1, "")
        out = b.ElementWiseNvrtc([y, rs], 1, code, 7, num_list_outputs=1)[0]
        b.Free(y)
        b.output("out", out)
        before = vm.counter("qlinearconv_residual_fusions")
        prog = vm.Program(b.serialize())
        got = prog.run({"x": g.to_channels_last(g.dev(x)), "r": g.to_channels_last(g.dev(r))})["out"]
        prog.close()
        assert vm.counter("qlinearconv_residual_fusions") - before == expect
        conv = oracle.qlinear_conv_int(x, 0.02, 128, w, ws, np.zeros(32, np.int8), np.float32(0.25), 120, np.uint8)
        s_ = oracle.binary(oracle.ADD, oracle.dequantize_linear(r, 0.1, 3), oracle.dequantize_linear(conv, group_scale, 120))
        np.testing.assert_array_equal(got, oracle.quantize_linear(s_, 0.3, 100, np.uint8))


def test_value_kept_minus_128_reaches_a_group_that_runs_unfused(g, vm, oracle):
    """A value only convolutions read is kept as code - 128; when the residual sum that reads it is, at run time, not
    the convolution's to compute after all (other constants), the group instruction gets plain codes back."""
    rng = np.random.default_rng(78)
    x = rand_q(rng, (2, 16, 6, 5), np.uint8)
    w0 = rng.integers(-127, 128, size=(32, 16, 1, 1)).astype(np.int8)
    w1 = rng.integers(-127, 128, size=(32, 32, 1, 1)).astype(np.int8)
    ws0 = rng.uniform(0.002, 0.01, size=32).astype(np.float32)
    ws1 = rng.uniform(0.002, 0.01, size=32).astype(np.float32)
    zeros = np.zeros(32, np.int8)
    u8 = torch.uint8

    def scale_bits(v):
        return "0x%08x" % np.float32(v).view(np.uint32)
    for group_scale, fused in ((0.25, 1), (0.26, 0)):
        code = g.ops.fusion_program(
            [("a", u8), ("b", u8)],
            [("fa", "DequantizeLinear", "a", scale_bits(group_scale), 120), ("fb", "DequantizeLinear", "b", scale_bits(0.1), 3),
             ("s", "Add", "fb", "fa"), ("q", "QuantizeLinear", "s", scale_bits(0.3), 100, "uint8")], [("q", u8)])
        b = vm.ProgramBuilder()
        xs = b.input("x", "uint8", x.shape)
        r = b.QLinearConv(xs, b.scalar(0.02, "float32"), b.scalar(128, "uint8"), b.constant(w0), b.constant(ws0), b.constant(zeros),
                          b.scalar(0.1, "float32"), b.scalar(3, "uint8"), None, [1, 1], [0, 0], 1, "")
        y = b.QLinearConv(r, b.scalar(0.1, "float32"), b.scalar(3, "uint8"), b.constant(w1), b.constant(ws1), b.constant(zeros),
                          b.scalar(0.25, "float32"), b.scalar(120, "uint8"), None, [1, 1], [0, 0], 1, "")
        out = b.ElementWiseNvrtc([y, r], 1, code, 7, num_list_outputs=1)[0]
        b.Free(y)
        b.Free(r)
        b.output("out", out)
        fusions, stores = vm.counter("qlinearconv_residual_fusions"), vm.counter("minus_128_stores")
        prog = vm.Program(b.serialize())
        got = prog.run({"x": g.to_channels_last(g.dev(x))})["out"]
        prog.close()
        assert vm.counter("qlinearconv_residual_fusions") - fusions == fused
        assert vm.counter("minus_128_stores") - stores == 1   # r; `out` is read by the caller
        rv = oracle.qlinear_conv_int(x, 0.02, 128, w0, ws0, zeros, np.float32(0.1), 3, np.uint8)
        conv = oracle.qlinear_conv_int(rv, 0.1, 3, w1, ws1, zeros, np.float32(0.25), 120, np.uint8)
        s_ = oracle.binary(oracle.ADD, oracle.dequantize_linear(rv, 0.1, 3), oracle.dequantize_linear(conv, group_scale, 120))
        np.testing.assert_array_equal(got, oracle.quantize_linear(s_, 0.3, 100, np.uint8))
    # with type checks on, the run keeps plain codes (the program's types say uint8)
    stores = vm.counter("minus_128_stores")
    prog = vm.Program(b.serialize())
    vm.set_option("check_types", "on")
    try:
        prog.run({"x": g.to_channels_last(g.dev(x))})
    finally:
        vm.set_option("check_types", "off")
    prog.close()
    assert vm.counter("minus_128_stores") == stores


def test_unfused_pools_run_as_float_ops(g, vm, oracle):
    """A MaxPool / AveragePool that is not between a DequantizeLinear and a QuantizeLinear is the float op of
    runtime/ops/pooling.cc:47-75; asking for its backward context is refused when the program is loaded."""
    rng = np.random.default_rng(21)
    xv = rng.standard_normal((2, 3, 9, 8)).astype(np.float32)
    b = vm.ProgramBuilder()
    x = b.input("x", "float32", xv.shape)
    y, a = b.new_slot(), b.new_slot()
    b.add_raw("MaxPool", [("ARRAY", x), ("INTS", [3, 2]), ("INTS", [2, 2]), ("INTS", [1, 0]), ("INT", 1), ("STRING", "NOTSET")], [y, -1])
    b.add_raw("AveragePool", [("ARRAY", x), ("INTS", [3, 3]), ("INTS", [2, 1]), ("INTS", [1, 1]), ("INT", 0)], [a, -1])
    b.output("y", y)
    b.output("a", a)
    prog = vm.Program(b.serialize())
    for xd in (g.dev(xv), g.to_channels_last(g.dev(xv))):
        out = prog.run({"x": xd})
        np.testing.assert_array_equal(out["y"], oracle.max_pool(xv, (3, 2), (2, 2), (1, 0), True))
        np.testing.assert_array_equal(out["a"].view(np.int32), oracle.average_pool(xv, (3, 3), (2, 1), (1, 1), False).view(np.int32))
    prog.close()
    b = vm.ProgramBuilder()
    x = b.input("x", "float32", (1, 1, 4, 4))
    y, c = b.new_slot(), b.new_slot()
    b.add_raw("MaxPool", [("ARRAY", x), ("INTS", [2, 2]), ("INTS", [2, 2]), ("INTS", [0, 0]), ("INT", 0), ("STRING", "NOTSET")], [y, c])
    b.output("y", y)
    with pytest.raises(vm.ChxVMError, match="backward context"):
        vm.Program(b.serialize())


def test_nan_and_inf_scans(g, vm, capsys):
    """check_nans / check_infs (runtime/chxvm_state.cc:202-263): off by default; when on, the first
    instruction whose result holds a NaN / an Inf fails the run and names its operands."""
    b = vm.ProgramBuilder()
    x = b.input("x", "uint8", (4, 6))
    d = b.DequantizeLinear(x, b.scalar(float("inf"), "float32"), b.scalar(3, "uint8"))   # (x - 3) * inf
    b.output("d", d)
    prog = vm.Program(b.serialize())
    xv = np.full((4, 6), 9, np.uint8)
    xv[2, 5] = 3                                            # 0 * inf = NaN
    try:
        out = prog.run({"x": g.dev(xv)})["d"]
        assert np.isnan(out[2, 5]) and np.isinf(out).sum() == 23
        vm.set_option("check_infs", "on")
        with pytest.raises(vm.ChxVMError, match=r"Inf detected!(.|\n)*input #0: uint8\(4, 6\)(.|\n)*output #0: float32\(4, 6\)"):
            prog.run({"x": g.dev(xv)})
        vm.set_option("check_infs", "off")
        vm.set_option("check_nans", "on")
        with pytest.raises(vm.ChxVMError, match="NaN detected!"):
            prog.run({"x": g.dev(xv)})
        xv[2, 5] = 4                                        # no NaN left: the NaN scan passes, Inf is not its business
        assert np.isinf(prog.run({"x": g.dev(xv)})["d"]).all()
        with pytest.raises(vm.ChxVMError, match="'on' or 'off'"):
            vm.set_option("check_nans", "1")
    finally:
        vm.set_option("check_nans", "off")
        vm.set_option("check_infs", "off")
        prog.close()


def test_count_nonfinite_entry_point(g):
    """chx_hip_count_nonfinite on dense and strided float32 arrays; other element types count 0."""
    import ctypes
    rng = np.random.default_rng(5)
    a = rng.standard_normal((37, 2, 129)).astype(np.float32)
    a[3, 1, 7] = np.nan
    a[36, 0, 128] = -np.nan
    a[0, 0, 0] = np.inf
    a[5, 1, 100] = -np.inf
    a[6, 1, 101] = np.inf
    a[7, 0, 1] = np.float32(3.4028235e38)                    # largest finite value: neither
    t = g.dev(a)

    def count(tensor, infinities):
        n = ctypes.c_int64(-1)
        g.capi.check(g.capi.lib().chx_hip_count_nonfinite(g.capi.ref(tensor), ctypes.c_int32(infinities), ctypes.byref(n), g.capi.stream_ptr()))
        return n.value
    assert (count(t, 0), count(t, 1)) == (2, 3)
    view = t[:, 1, ::2]                                      # strided: row 1 of every pair, even columns
    assert (count(view, 0), count(view, 1)) == (int(np.isnan(a[:, 1, ::2]).sum()), int(np.isinf(a[:, 1, ::2]).sum())) == (0, 1)
    assert count(g.dev(np.arange(12, dtype=np.int32)), 0) == 0 and count(t[:0], 1) == 0
    big = torch.zeros(3_000_001, device="cuda")
    big[::1000] = float("inf")
    assert count(big, 1) == 3001 and count(big, 0) == 0


def test_trace_lines(g, vm, capfd):
    """trace_level 1 prints, per instruction, the lines of the reference's generated glue
    (runtime/gen_chxvm.py:190-236,309-318): "$out = Op($in, ...)", the array operands' dtype and shape,
    " ->", the results' dtype and shape."""
    import re
    b = vm.ProgramBuilder()
    x = b.input("x", "float32", (3, 5))
    q = b.QuantizeLinear(x, b.scalar(0.5, "float32"), None, debug_info="the quantization")
    b.output("q", q)
    prog = vm.Program(b.serialize())
    capfd.readouterr()
    prog.run({"x": g.dev(np.ones((3, 5), np.float32))}, trace_level=1)
    err = capfd.readouterr().err
    prog.close()
    assert re.search(r"^# the quantization\n\$%d = QuantizeLinear\(\$%d, \$\d+, \$-1\)\n \$%d=float32\(3, 5\) -> \$%d=uint8\(3, 5\)$" % (q, x, x, q),
                     err, flags=re.M), err
    assert re.search(r'^\$%d = In\("?name"?\)\n' % x, err, flags=re.M) and re.search(r"^Out\(.*\$%d\)$" % q, err, flags=re.M), err
    prog = vm.Program(b.serialize())
    prog.run({"x": g.dev(np.ones((3, 5), np.float32))})          # silent by default
    assert capfd.readouterr().err == ""
    prog.close()


def test_max_pool_on_codes_for_both_8_bit_types(g, vm, oracle):
    """DequantizeLinear -> MaxPool -> QuantizeLinear with one scale and zero point runs as one kernel on the
    codes: the maximum for uint8 (Q(DQ(q)) == q); for int8 the reference's truncating QuantizeLinear gives
    q + 1 for a negative q, and so does the kernel.  Checked against the three float ops of the oracle."""
    def pool_program(zp, zdt):
        b = vm.ProgramBuilder()
        x = b.input("x", zdt, (1, 16, 6, 6))
        s, z = b.scalar(0.05, "float32"), b.scalar(zp, zdt)
        d = b.DequantizeLinear(x, s, z)
        p = b.new_slot()
        b.add_raw("MaxPool", [("ARRAY", d), ("INTS", [2, 2]), ("INTS", [2, 2]), ("INTS", [0, 0]), ("INT", 0), ("STRING", "NOTSET")], [p, -1])
        q = b.QuantizeLinear(p, s, z)
        b.output("q", q)
        return b.serialize()
    rng = np.random.default_rng(8)
    for dt, zp in ((np.uint8, 30), (np.int8, -3)):
        info = np.iinfo(dt)
        x = rng.integers(info.min, info.max + 1, size=(1, 16, 6, 6)).astype(dt)
        prog = vm.Program(pool_program(zp, np.dtype(dt).name))
        got = prog.run({"x": g.dev(x)})["q"]
        prog.close()
        np.testing.assert_array_equal(got, oracle.max_pool_q8(x, (2, 2), (2, 2)))
        pooled = oracle.dequantize_linear(x, np.float32(0.05), zp).reshape(1, 16, 3, 2, 3, 2).max(axis=(3, 5))
        np.testing.assert_array_equal(got, oracle.quantize_linear(pooled, np.float32(0.05), zp, dt))
        if dt == np.int8:
            m = x.reshape(1, 16, 3, 2, 3, 2).max(axis=(3, 5)).astype(np.int64)
            assert (m < 0).any()
            np.testing.assert_array_equal(got, m + (m < 0))


def _conv_program(vm, shape, w, ws, wz, bias, xq, yq, weights_as_inputs=False):
    """QuantizeLinear -> QLinearConv -> Out; the four weight-side operands constants or program inputs."""
    b = vm.ProgramBuilder()
    x = b.input("x", "float32", shape)
    s_x, z_x = b.scalar(float(xq[0]), "float32"), b.scalar(int(xq[1]), "uint8")
    q = b.QuantizeLinear(x, s_x, z_x)
    if weights_as_inputs:
        ops = [b.input("w", "int8", w.shape), b.input("w_scale", "float32", ws.shape), b.input("w_zero_point", "int8", wz.shape),
               b.input("bias", "int32", bias.shape)]
    else:
        ops = [b.constant(w), b.constant(ws), b.constant(wz), b.constant(bias)]
    y = b.QLinearConv(q, s_x, z_x, ops[0], ops[1], ops[2], b.scalar(float(yq[0]), "float32"), b.scalar(int(yq[1]), "uint8"), ops[3],
                      [1, 1], [1, 1], 1, "")
    b.Free(q)
    b.output("y", y)
    return vm.Program(b.serialize())


def test_two_programs_keep_their_own_bias_mode(g, vm, oracle):
    """The bias mode of a QLinearConv is an option of the run, not of the process: two programs with
    different settings, run alternately, each give the result of their own mode."""
    rng = np.random.default_rng(21)
    N, C, H, W, OC = 2, 32, 8, 9, 64
    w = rng.integers(-127, 128, size=(OC, C, 3, 3)).astype(np.int8)
    ws = rng.uniform(0.001, 0.01, size=OC).astype(np.float32)
    wz = np.zeros(OC, np.int8)
    bias = rng.integers(-3000, 3000, size=OC).astype(np.int32)
    xq, yq = (np.float32(0.02), 128), (np.float32(0.2), 100)
    p_ref = _conv_program(vm, (N, C, H, W), w, ws, wz, bias, xq, yq)
    p_onnx = _conv_program(vm, (N, C, H, W), w, ws, wz, bias, xq, yq)
    p_onnx.set_option("qlinearconv_bias", "onnx_int32")
    p_ref.set_option("qlinearconv_bias", "reference")
    xv = rng.uniform(-2.5, 2.5, size=(N, C, H, W)).astype(np.float32)
    qx = oracle.quantize_linear(xv, xq[0], xq[1], np.uint8)
    want = {mode: oracle.qlinear_conv_int(qx, xq[0], xq[1], w, ws, wz, yq[0], yq[1], np.uint8, bias=bias, bias_mode=mode,
                                          strides=(1, 1), pads=(1, 1)) for mode in (oracle.BIAS_REFERENCE_FLOAT, oracle.BIAS_ONNX_INT32)}
    assert (want[oracle.BIAS_REFERENCE_FLOAT] != want[oracle.BIAS_ONNX_INT32]).any()
    for _ in range(2):
        np.testing.assert_array_equal(p_ref.run({"x": g.dev(xv)})["y"], want[oracle.BIAS_REFERENCE_FLOAT])
        np.testing.assert_array_equal(p_onnx.run({"x": g.dev(xv)})["y"], want[oracle.BIAS_ONNX_INT32])
    # "default" follows the process-wide switch again
    p_onnx.set_option("qlinearconv_bias", "default")
    np.testing.assert_array_equal(p_onnx.run({"x": g.dev(xv)})["y"], want[oracle.BIAS_REFERENCE_FLOAT])
    with pytest.raises(vm.ChxVMError, match="unknown program option"):
        p_ref.set_option("no_such_option", "on")


def test_weights_that_are_program_inputs_are_read_on_every_run(g, vm, oracle):
    """Weight-side operands that come from the caller get no cached plan: a second run with other weights at
    the same device addresses (rewritten in place) computes with the new ones."""
    rng = np.random.default_rng(22)
    N, C, H, W, OC = 1, 64, 7, 7, 64
    xq, yq = (np.float32(0.02), 128), (np.float32(0.15), 128)
    xv = rng.uniform(-2.5, 2.5, size=(N, C, H, W)).astype(np.float32)
    qx = oracle.quantize_linear(xv, xq[0], xq[1], np.uint8)
    shapes = ((OC, C, 3, 3), (OC,), (OC,), (OC,))
    prog = _conv_program(vm, (N, C, H, W), np.zeros(shapes[0], np.int8), np.zeros(OC, np.float32), np.zeros(OC, np.int8),
                         np.zeros(OC, np.int32), xq, yq, weights_as_inputs=True)
    dev = {"w": torch.zeros(shapes[0], dtype=torch.int8, device="cuda"), "w_scale": torch.zeros(OC, dtype=torch.float32, device="cuda"),
           "w_zero_point": torch.zeros(OC, dtype=torch.int8, device="cuda"), "bias": torch.zeros(OC, dtype=torch.int32, device="cuda")}
    seen = []
    for seed in (1, 2, 3):
        r = np.random.default_rng(seed)
        w = r.integers(-127, 128, size=shapes[0]).astype(np.int8)
        ws = r.uniform(0.001, 0.01, size=OC).astype(np.float32)
        bias = r.integers(-5, 6, size=OC).astype(np.int32)
        dev["w"].copy_(torch.from_numpy(w))           # the same device memory, new contents
        dev["w_scale"].copy_(torch.from_numpy(ws))
        dev["bias"].copy_(torch.from_numpy(bias))
        torch.cuda.synchronize()
        got = prog.run(dict(dev, x=g.dev(xv)))["y"]
        want = oracle.qlinear_conv_int(qx, xq[0], xq[1], w, ws, np.zeros(OC, np.int8), yq[0], yq[1], np.uint8, bias=bias,
                                       bias_mode=oracle.BIAS_REFERENCE_FLOAT, strides=(1, 1), pads=(1, 1))
        np.testing.assert_array_equal(got, want)
        seen.append(got)
    assert (seen[0] != seen[1]).any() and (seen[1] != seen[2]).any()


def test_type_checks_and_dumps_of_a_program_with_fused_instructions(g, vm, oracle, tmp_path):
    """A compiled network: pools (two outputs, the second the dropped context), QLinearConv with the residual
    group behind it computed inside, DequantizeLinear absorbed into pools.  With the run-time type check on
    and every named output dumped, the instructions that were fused away (their named outputs stay unset)
    are skipped, everything else is checked and written."""
    from importlib import import_module
    onnx_lite = import_module(g.pkg.__name__ + ".onnx_lite")
    wl = g.pkg.workloads
    model = wl.build_resnet50(batch=2, image=64, seed=5, width=16, blocks=(1, 1, 1, 1), classes=10)
    data = vm.compile_onnx(wl.program_to_onnx(model, onnx_lite), {"fuse": "hip"})
    prog = vm.Program(data)
    prog.set_option("qlinearconv_bias", "onnx_int32")
    before = prog.counter("qlinearconv_residual_fusions")
    vm.set_option("check_types", "on")
    vm.set_option("dump_outputs_dir", str(tmp_path))
    try:
        got = prog.run({"x": torch.from_numpy(model["input"]).cuda()})["logits"]
    finally:
        vm.set_option("check_types", "off")
        vm.set_option("dump_outputs_dir", "")
    assert prog.counter("qlinearconv_residual_fusions") - before == 4
    oracle.set_threads(16)
    try:
        ref = wl.run_reference(model, oracle, model["input"], keep={"logits"})
    finally:
        oracle.set_threads(1)
    np.testing.assert_array_equal(got, ref["logits"])
    dumped = sorted(p.name for p in tmp_path.iterdir())
    assert len(dumped) > 10 and any(name.endswith("logits.npy") for name in dumped)
    last = [p for p in tmp_path.iterdir() if p.name.endswith("logits.npy")][0]
    np.testing.assert_array_equal(np.load(last), ref["logits"])


def test_recorded_run_replays_with_new_inputs(g, vm, oracle):
    """A program recorded into a device graph: every replay (with eager work and synchronizations of the
    program's own in between) gives the oracle's values for what the input buffer holds at that time."""
    wl = g.pkg.workloads
    for model in (wl.build_resnet50(batch=2, image=64, seed=5, width=16, blocks=(2, 1, 1, 1), classes=10),
                  wl.build_mobilenetv2(batch=2, image=64, seed=7, blocks=((1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 1, 2)), stem=32,
                                       head=128, classes=10)):
        keep = ["logits"] + [ins[1] for ins in model["program"] if ins[0] in ("AddRelu", "Add")]
        prog = vm.Program(wl.program_to_chxvm(model, vm, g.pkg.ops, keep=keep).serialize())
        prog.set_option("qlinearconv_bias", "onnx_int32")
        x = torch.from_numpy(model["input"]).cuda()
        replay = prog.capture({"x": x})
        assert replay.info("warm_runs") >= 2 and replay.info("pool_bytes") > 0
        rng = np.random.default_rng(9)
        oracle.set_threads(16)
        try:
            for i in range(4):
                xv = model["input"] if i == 0 else (model["input"] * np.float32(0.5 + 0.25 * i) +
                                                    rng.standard_normal(model["input"].shape).astype(np.float32) * np.float32(0.3))
                x.copy_(torch.from_numpy(xv))
                torch.cuda.synchronize()
                replay.launch()
                replay.synchronize()
                got = replay.outputs()
                ref = wl.run_reference(model, oracle, xv, keep=set(keep))
                for name in keep:
                    np.testing.assert_array_equal(got[name], ref[name], err_msg="replay %d value %s" % (i, name))
                # eager work of the same program between the replays (its plans and kernels are shared)
                eager = prog.run({"x": x})
                np.testing.assert_array_equal(eager["logits"], ref["logits"])
        finally:
            oracle.set_threads(1)
        # launched on the caller's stream as well
        replay.launch(g.capi.stream_ptr())
        torch.cuda.synchronize()
        np.testing.assert_array_equal(replay.outputs()["logits"], ref["logits"])
        replay.close()
        prog.close()


def test_recorded_integer_ops_follow_the_input(g, vm, oracle):
    """ConvInteger and MatMulInteger inside a recorded run: they are launched on the recording stream like every
    other op, so each replay computes them from what the input buffers hold then (on the null stream they would
    run once while recording, and every replay would return those first results)."""
    rng = np.random.default_rng(21)
    x, w = rand_q(rng, (2, 32, 9, 8), np.uint8), rand_q(rng, (16, 32, 3, 3), np.int8)
    a_, b_ = rand_q(rng, (24, 64), np.uint8), rand_q(rng, (64, 40), np.int8)
    b = vm.ProgramBuilder()
    xi = b.input("x", "uint8", x.shape)
    b.output("y", b.ConvInteger(xi, b.constant(w), b.scalar(77, "uint8"), None, [1, 1], [1, 1], 1, ""))
    ai = b.input("a", "uint8", a_.shape)
    b.output("m", b.MatMulInteger(ai, b.constant(b_), b.constant(np.array([3], np.uint8)), None))
    prog = vm.Program(b.serialize())
    xd, ad = g.dev(x), g.dev(a_)
    replay = prog.capture({"x": xd, "a": ad})
    for i in range(3):
        xv, av = rand_q(rng, x.shape, np.uint8), rand_q(rng, a_.shape, np.uint8)
        xd.copy_(torch.from_numpy(xv))
        ad.copy_(torch.from_numpy(av))
        torch.cuda.synchronize()
        replay.launch()
        replay.synchronize()
        got = replay.outputs()
        np.testing.assert_array_equal(got["y"], oracle.conv_integer(xv, w, 77, None, strides=(1, 1), pads=(1, 1), group=1),
                                      err_msg="replay %d" % i)
        np.testing.assert_array_equal(got["m"], oracle.matmul_integer(av, b_, np.array([3], np.uint8), None), err_msg="replay %d" % i)
    replay.close()
    prog.close()


def test_a_program_that_reads_results_back_cannot_be_recorded(g, vm):
    """A dynamically quantized graph computes its scales on the device and reads them back as scalars: the
    capture fails with the reason, and the program still runs eagerly afterwards."""
    b = vm.ProgramBuilder()
    x = b.input("x", "float32", (4, 64))
    lo = b.ReduceMin(x, [], 0)
    s = b.new_slot()
    b.add_raw("Identity", [("ARRAY", lo)], [s])
    q = b.QuantizeLinear(x, b.scalar(0.05, "float32"), b.scalar(3, "uint8"))
    b.output("q", q)
    b.output("lo", lo)
    prog = vm.Program(b.serialize())
    xv = np.random.default_rng(3).standard_normal((4, 64)).astype(np.float32)
    xd = g.dev(xv)
    try:
        replay = prog.capture({"x": xd})
    except vm.ChxVMError as e:
        assert "capture" in str(e) or "captur" in str(e) or "graph" in str(e)
    else:
        # the reduction itself needs no read-back in this build: then the replay must be right
        replay.launch()
        replay.synchronize()
        assert np.float32(replay.outputs()["lo"]) == xv.min()
        replay.close()
    out = prog.run({"x": xd})
    assert np.float32(out["lo"]) == xv.min()


@pytest.mark.parametrize("net,batch,seed", [("resnet50", 64, 3), ("mobilenetv2", 128, 4)])
def test_benchmark_networks_at_full_size_through_the_vm(g, vm, oracle, net, batch, seed):
    """What bench.py times by default: the whole network at its benchmark batch as one serialized program in the
    C++ VM, its run recorded and replayed.  Three images of the batch are compared with the oracle on the
    logits and on every block output; all images through the property that needs no oracle (every op of the
    path is independent per image, so a permuted batch gives the permuted results)."""
    wl = g.pkg.workloads
    model = (wl.build_resnet50 if net == "resnet50" else wl.build_mobilenetv2)(batch=batch, seed=seed)
    keep = ["logits"] + [ins[1] for ins in model["program"] if ins[0] in ("AddRelu", "Add")]
    prog = vm.Program(wl.program_to_chxvm(model, vm, g.pkg.ops, keep=keep).serialize())
    prog.set_option("qlinearconv_bias", "onnx_int32")
    x = torch.from_numpy(model["input"]).cuda()
    replay = prog.capture({"x": x})
    fused = prog.counter("qlinearconv_residual_fusions")
    assert fused >= len(keep) - 1          # every residual sum was computed inside its convolution, in every run
    replay.launch()
    replay.synchronize()
    out = replay.outputs()
    picks = [0, batch // 2 + 5, batch - 1]
    oracle.set_threads(16)
    try:
        ref = wl.run_reference(model, oracle, model["input"][picks], keep=set(keep))
    finally:
        oracle.set_threads(1)
    for name in keep:
        np.testing.assert_array_equal(out[name][picks], ref[name], err_msg=name)
    assert out["logits"].min() < out["logits"].max()
    perm = torch.randperm(batch, generator=torch.Generator().manual_seed(seed))
    x.copy_(x[perm.cuda()])
    torch.cuda.synchronize()
    replay.launch(g.capi.stream_ptr())
    torch.cuda.synchronize()
    again = replay.outputs()
    for name in keep:
        np.testing.assert_array_equal(again[name], out[name][perm.numpy()], err_msg=name)
    replay.close()
    prog.close()


def test_fusion_group_with_the_reference_kernel_text(g, vm, oracle):
    """An ElementWiseNvrtc instruction whose `code` is the CUDA C text that the reference's compiler emits (the group of
    compiler/fusion_test.cc, Tanh -> Sigmoid): it loads and runs; the sigmoid is that text's helper."""
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "nvrtc_fusion_sources.json")) as f:
        src = json.load(f)
    b = vm.ProgramBuilder()
    (y,) = b.ElementWiseNvrtc([b.input("input")], 1, src["tanh_sigmoid_float"], 1, num_list_outputs=1)
    b.output("output", y)
    prog = vm.Program(b.serialize())
    x = (np.random.default_rng(41).standard_normal((2, 50, 30)) * 3).astype(np.float32)
    out = prog.run({"input": g.dev(x)})
    np.testing.assert_array_equal(out["output"], oracle.sigmoid_tanh_form(oracle.tanh(x)))
    # in half precision the results are float16 arrays
    bh = vm.ProgramBuilder()
    (yh,) = bh.ElementWiseNvrtc([bh.input("x", "float16"), bh.input("a", "float16"), bh.input("b", "float16"), bh.input("c", "float16")], 1,
                                src["chain_T"].replace("@T@", "half"), 3, num_list_outputs=1)
    bh.output("y", yh)
    xs = [torch.from_numpy(np.random.default_rng(42 + i).standard_normal((4, 16)).astype(np.float16)).cuda() for i in range(4)]
    out = vm.Program(bh.serialize()).run(dict(zip("xabc", xs)))
    assert out["y"].dtype == np.float16 and out["y"].shape == (4, 16)


def test_bit_shift_instruction(g, vm):
    """BitShift as a VM instruction (IDL row of runtime/chxvm_defs.py:471): direction is a string attribute."""
    x = np.arange(24, dtype=np.uint8).reshape(2, 3, 4) * 9
    y = np.array([1, 0, 3, 7], np.uint8)
    for direction, fn in (("LEFT", np.left_shift), ("RIGHT", np.right_shift)):
        b = vm.ProgramBuilder()
        b.output("z", b.BitShift(b.input("x", "uint8"), b.constant(y), direction))
        out = vm.Program(b.serialize()).run({"x": g.dev(x)})
        np.testing.assert_array_equal(out["z"], fn(x, y))
    b = vm.ProgramBuilder()
    b.output("z", b.BitShift(b.input("x", "uint8"), b.constant(y), "UP"))
    with pytest.raises(vm.ChxVMError) as e:
        vm.Program(b.serialize()).run({"x": g.dev(x)})
    assert "direction" in str(e.value)


def test_convolution_over_one_spatial_axis_as_an_instruction(g, vm, oracle):
    """QLinearConv and ConvInteger on x [N,C,L]: the attributes are completed for one spatial axis
    (ComplementStride / ComplementPad, runtime/chainerx_util.cc:180-200) and the result has three axes."""
    rng = np.random.default_rng(71)
    x, w = rand_q(rng, (2, 64, 40), np.uint8), rand_q(rng, (16, 64, 3), np.int8)
    ws, wz = rng.uniform(0.001, 0.01, 16).astype(np.float32), np.zeros(16, np.int8)
    b = vm.ProgramBuilder()
    xi = b.input("x", "uint8", x.shape)
    y = b.QLinearConv(xi, b.scalar(0.02, "float32"), b.scalar(3, "uint8"), b.constant(w), b.constant(ws), b.constant(wz),
                      b.scalar(0.05, "float32"), b.scalar(128, "uint8"), None, [], [1], 1, "")
    b.output("y", y)
    b.output("yi", b.ConvInteger(xi, b.constant(w), b.scalar(3, "uint8"), None, [2], [], 1, ""))
    out = vm.Program(b.serialize()).run({"x": g.dev(x)})
    want = oracle.qlinear_conv_int(x[:, :, None, :], 0.02, 3, w[:, :, None, :], ws, wz, 0.05, 128, np.uint8, strides=(1, 1), pads=(0, 1))
    np.testing.assert_array_equal(out["y"], want[:, :, 0, :])
    np.testing.assert_array_equal(out["yi"], oracle.conv_integer(x[:, :, None, :], w[:, :, None, :], 3, None, strides=(1, 2), pads=(0, 0))[:, :, 0, :])


def test_a_recording_pins_the_plans_it_has_used(g, vm, oracle):
    """The kernels of a recorded run address the scratch memory of the convolution plans.  An eager run of the same
    program on a larger input, which would have to move that memory, is refused while the recording lives; the
    recording keeps giving the right values, and after its destruction the larger run goes through."""
    rng = np.random.default_rng(81)
    w = rand_q(rng, (32, 64, 3, 3), np.int8)
    ws, wz = rng.uniform(0.001, 0.01, 32).astype(np.float32), np.zeros(32, np.int8)
    b = vm.ProgramBuilder()
    y = b.QLinearConv(b.input("x", "uint8"), b.scalar(0.02, "float32"), b.scalar(0, "uint8"), b.constant(w), b.constant(ws), b.constant(wz),
                      b.scalar(0.05, "float32"), b.scalar(128, "uint8"), None, [], [1, 1], 1, "")
    b.output("y", y)
    prog = vm.Program(b.serialize())
    small, large = rand_q(rng, (1, 64, 12, 12), np.uint8), rand_q(rng, (4, 64, 20, 20), np.uint8)
    want = lambda x: oracle.qlinear_conv_int(x, 0.02, 0, w, ws, wz, 0.05, 128, np.uint8, pads=(1, 1))
    xd = g.dev(small)   # NCHW-contiguous: the plan transposes it into scratch memory of its own
    replay = prog.capture({"x": xd})
    with pytest.raises(vm.ChxVMError) as e:
        prog.run({"x": g.dev(large)})
    assert "pinned by a recorded run" in str(e.value)
    again = rand_q(rng, small.shape, np.uint8)
    xd.copy_(torch.from_numpy(again))
    torch.cuda.synchronize()
    replay.launch()
    replay.synchronize()
    np.testing.assert_array_equal(replay.outputs()["y"], want(again))
    np.testing.assert_array_equal(prog.run({"x": g.dev(small)})["y"], want(small))   # the recorded size still runs eagerly
    replay.close()
    np.testing.assert_array_equal(prog.run({"x": g.dev(large)})["y"], want(large))
    prog.close()
