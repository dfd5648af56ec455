"""Fused element-wise chains on the MI355X through the C ABI against the op-by-op
CPU oracle (compiler/chxvm/emitter.cc:697-726: on the CPU a FusionGroup runs as its
individual ops, one fp32 rounding each).

Tolerance: the requirement is 2 ulp or 1e-6 relative per element.  The device code
reproduces the host C library's tanhf/expf operation by operation, so the tests
assert the stronger property, bit equality, and state the tolerance where a looser
comparison is made on purpose."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

F32 = torch.float32
ULP_TOL = 2
REL_TOL = 1e-6


@pytest.fixture(scope="module")
def g():
    import gpu_util
    gpu_util.capi.init(0)
    return gpu_util


def chain_program(ops):
    return ops.fusion_program(
        [("x", F32), ("a", F32), ("b", F32), ("c", F32)],
        [("t0", "Mul", "x", "a"), ("t1", "Add", "t0", "b"), ("t2", "Tanh", "t1"), ("t3", "Sigmoid", "c"),
         ("t4", "Mul", "t2", "t3"), ("t5", "Add", "t4", "x"), ("y", "Relu", "t5")],
        [("y", F32)])


ORACLE_CHAIN = [("t0", "Mul", "x", "a"), ("t1", "Add", "t0", "b"), ("t2", "Tanh", "t1"), ("t3", "Sigmoid", "c"),
                ("t4", "Mul", "t2", "t3"), ("t5", "Add", "t4", "x"), ("y", "Relu", "t5")]


def within_tolerance(got, want):
    ulp = np.abs(got.view(np.int32).astype(np.int64) - want.view(np.int32).astype(np.int64))
    rel = np.abs(got.astype(np.float64) - want) <= REL_TOL * np.abs(want.astype(np.float64))
    return (ulp <= ULP_TOL) | rel | (got == want)


def unary_program(ops, op):
    return ops.fusion_program([("x", F32)], [("y", op, "x")], [("y", F32)])


@pytest.mark.parametrize("op", ["Tanh", "Exp", "Sigmoid"])
def test_transcendentals_bit_exact_over_every_float(g, oracle, op):
    """Every fp32 bit pattern, all 2^32 of them, against the host C library (in chunks of 2^26; about 15 s per
    function with the host side on all cores).  The device code of tanhf and of the sigmoid divides with a short
    sequence that is valid because this test says so (div_in_range in csrc/faithful_math.h), hence no sampling.
    CHX_FM_DEVICE_STRIDE=n in the environment takes every n-th pattern plus the neighbourhoods where the
    algorithms switch branches."""
    import os
    stride = int(os.environ.get("CHX_FM_DEVICE_STRIDE", "1"))
    edges = np.array([0x3f800000, 0x41b00000, 0x24000000, 0x3eb17218, 0x3F851592, 0x33000000, 0x4195b844,
                      0x42b17218, 0x42b00000, 0x42cff1b5, 0x4202422f, 0xc27c65d9, 0x7f800000, 0x00800000,
                      0x7e800000, 0x7e000000, 0xc2ad0000, 0xc2ae0000],
                     dtype=np.uint32)
    near = (edges[:, None].astype(np.int64) + np.arange(-64, 65)[None, :]).astype(np.uint32).reshape(-1)
    fn = {"Tanh": oracle.tanh, "Exp": oracle.exp, "Sigmoid": oracle.sigmoid}[op]
    prog = unary_program(g.ops, op)
    threads = oracle.max_threads() if stride < 16 else 1
    oracle.set_threads(threads)
    try:
        chunk = (1 << 26) * stride
        total = 0
        for lo in range(0, 1 << 32, chunk):
            bits = np.arange(lo, min(lo + chunk, 1 << 32), stride, dtype=np.uint64).astype(np.uint32)
            if lo == 0:
                bits = np.concatenate([bits, near, near | np.uint32(0x80000000)])
            x = bits.view(np.float32)
            want = fn(x)
            got = g.host(g.ops.ElementWiseNvrtc([g.dev(x)], 1, prog)[0])
            nan = np.isnan(want)
            assert np.array_equal(np.isnan(got), nan)
            mism = (got.view(np.uint32) != want.view(np.uint32)) & ~nan
            assert mism.sum() == 0, "%d of %d differ, first x=%r" % (mism.sum(), x.size, x[mism][:4])
            total += x.size
        assert total >= (1 << 32) // stride
    finally:
        oracle.set_threads(1)


@pytest.mark.parametrize("op", ["Exp", "Sigmoid", "chain"])
@pytest.mark.parametrize("share", [0.0005, 0.02, 0.5])
def test_rare_arguments_scattered_among_ordinary_ones(g, oracle, op, share):
    """The kernels evaluate a step's elements without expf's out-of-range cases and the sigmoid's near-denormal
    quotients first and repeat the step in full when any lane of the wavefront met one: so arguments of both kinds
    share wavefronts here (a few, some, half of the lanes), in the vector kernel and in the strided one."""
    rng = np.random.default_rng(int(share * 1e4) + len(op))
    n = 1 << 18
    x = (rng.standard_normal(n) * 3).astype(np.float32)
    rare = np.array([np.inf, -np.inf, np.nan, 88.0, -88.0, 88.5, 88.72283, 88.72284, 89.0, 100.0, 1e30, -86.6, -86.7, -87.0,
                     -87.4, -88.0, -100.0, -103.9, -103.98, -104.5, -150.0, -1e30, 86.6, 87.0, 87.4, 103.9, 104.5],
                    dtype=np.float32)
    at = rng.random(n) < share
    x[at] = rng.choice(rare, int(at.sum()))
    if op == "chain":
        c = x
        xx = rng.standard_normal(n).astype(np.float32)
        a, b = rng.standard_normal(256).astype(np.float32), rng.standard_normal(256).astype(np.float32)
        xx2, c2 = xx.reshape(-1, 256), c.reshape(-1, 256)
        want = oracle.run_chain(ORACLE_CHAIN, dict(x=xx2, a=a, b=b, c=c2))["y"]
        got = g.host(g.ops.ElementWiseNvrtc([g.dev(xx2), g.dev(a), g.dev(b), g.dev(c2)], 1, chain_program(g.ops), 3)[0])
        cases = [(got, want)]
    else:
        fn = {"Exp": oracle.exp, "Sigmoid": oracle.sigmoid}[op]
        prog = unary_program(g.ops, op)
        got = g.host(g.ops.ElementWiseNvrtc([g.dev(x)], 1, prog)[0])
        # every other element of a twice as long array: not contiguous, so the strided kernel runs
        wide = g.dev(np.repeat(x, 2))
        got2 = g.host(g.ops.ElementWiseNvrtc([wide[::2]], 1, prog)[0])
        cases = [(got, fn(x)), (got2, fn(x))]
    for got, want in cases:
        nan = np.isnan(want)
        assert np.array_equal(np.isnan(got), nan)
        assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])


@pytest.mark.parametrize("shape,vec_shape", [((8, 64, 256), (256,)), ((3, 5, 7), (7,)), ((2, 1000), (1000,)),
                                            ((1, 4), (4,)), ((5,), (1,))])
def test_chain_matches_oracle(g, oracle, shape, vec_shape):
    rng = np.random.default_rng(11)
    x = rng.standard_normal(shape).astype(np.float32)
    c = rng.standard_normal(shape).astype(np.float32)
    a = rng.standard_normal(vec_shape).astype(np.float32)
    b = rng.standard_normal(vec_shape).astype(np.float32)
    want = oracle.run_chain(ORACLE_CHAIN, dict(x=x, a=a, b=b, c=c))["y"]
    got = g.host(g.ops.ElementWiseNvrtc([g.dev(x), g.dev(a), g.dev(b), g.dev(c)], 1, chain_program(g.ops), 3)[0])
    assert got.shape == want.shape
    assert within_tolerance(got, want).all()          # the stated requirement
    np.testing.assert_array_equal(got, want)          # what the implementation actually delivers


def test_general_broadcast_and_multiple_outputs(g, oracle):
    rng = np.random.default_rng(12)
    x = rng.standard_normal((6, 1, 33)).astype(np.float32)
    col = rng.standard_normal((1, 9, 1)).astype(np.float32)   # broadcasts on the outer AND the inner axis
    prog = g.ops.fusion_program([("x", F32), ("k", F32)],
                                [("h", "Const", 0.5), ("s", "Sub", "x", "k"), ("e", "Exp", "s"), ("d", "Div", "e", "h"),
                                 ("m", "Max", "d", "x"), ("n", "Neg", "m"), ("cl", "Clip", "n", -3.0, 0.25)],
                                [("d", F32), ("cl", F32)])
    d, cl = g.ops.ElementWiseNvrtc([g.dev(x), g.dev(col)], 2, prog, 4)
    env = oracle.run_chain([("s", "Sub", "x", "k"), ("e", "Exp", "s")], dict(x=x, k=col))
    want_d = oracle.binary(oracle.DIV, env["e"], np.float32(0.5))
    want_cl = oracle.clip(-np.maximum(want_d, np.broadcast_to(x, want_d.shape)), -3.0, 0.25)
    assert d.shape == (6, 9, 33)
    np.testing.assert_array_equal(g.host(d), want_d)
    np.testing.assert_array_equal(g.host(cl), want_cl)


def test_quantized_residual_add_relu(g, oracle):
    """DequantizeLinear x2 -> Add -> Relu -> QuantizeLinear as one kernel on uint8 tensors, NCHW and
    channels-last."""
    rng = np.random.default_rng(13)
    qa = rng.integers(0, 256, size=(2, 24, 9, 9)).astype(np.uint8)
    qb = rng.integers(0, 256, size=(2, 24, 9, 9)).astype(np.uint8)
    prog = g.ops.fusion_program(
        [("qa", torch.uint8), ("qb", torch.uint8)],
        [("a", "DequantizeLinear", "qa", 0.05, 128), ("b", "DequantizeLinear", "qb", 0.02, 120),
         ("s", "Add", "a", "b"), ("r", "Relu", "s"), ("q", "QuantizeLinear", "r", 0.06, 3, "uint8")],
        [("q", torch.uint8)])
    s = oracle.binary(oracle.ADD, oracle.dequantize_linear(qa, 0.05, 128), oracle.dequantize_linear(qb, 0.02, 120))
    want = oracle.quantize_linear(oracle.relu(s), 0.06, 3, np.uint8)
    got = g.ops.ElementWiseNvrtc([g.dev(qa), g.dev(qb)], 1, prog, 5)[0]
    np.testing.assert_array_equal(g.host(got), want)
    cl = g.ops.ElementWiseNvrtc([g.to_channels_last(g.dev(qa)), g.to_channels_last(g.dev(qb))], 1, prog, 5)[0]
    assert cl.stride() == g.to_channels_last(g.dev(qa)).stride()
    np.testing.assert_array_equal(g.host(cl), want)


def test_fused_quantize_dequantize_round_trip(g, oracle):
    rng = np.random.default_rng(14)
    x = (rng.standard_normal((4, 1024)) * 3).astype(np.float32)
    prog = g.ops.fusion_program([("x", F32)], [("q", "QuantizeLinear", "x", 0.05, 0, "int8"),
                                               ("y", "DequantizeLinear", "q", 0.05, 0)], [("y", F32)])
    got = g.host(g.ops.ElementWiseNvrtc([g.dev(x)], 1, prog, 6)[0])
    np.testing.assert_array_equal(got, oracle.dequantize_linear(oracle.quantize_linear(x, 0.05, 0, np.int8), 0.05, 0))


def test_full_size_fused_quantize_dequantize(g, oracle):
    """The fused QuantizeLinear -> DequantizeLinear group on [64,1024,1024] (int8, scale 0.05, zero point 0), the kernel
    the benchmark times: sampled rows against the oracle, every element against the two separate kernels and through
    properties that need no oracle."""
    torch.manual_seed(1)
    x = torch.randn(64, 1024, 1024, device="cuda")
    prog = g.ops.fusion_program([("x", F32)], [("q", "QuantizeLinear", "x", 0.05, 0, "int8"),
                                               ("y", "DequantizeLinear", "q", 0.05, 0)], [("y", F32)])
    y = g.ops.ElementWiseNvrtc([x], 1, prog, 3)[0]
    torch.cuda.synchronize()
    assert y.shape == x.shape and y.dtype == torch.float32
    # the two ops as kernels of their own give the same bits
    assert torch.equal(y, g.ops.DequantizeLinear(g.ops.QuantizeLinear(x, 0.05, 0, torch.int8), 0.05, 0))
    # every result is a code times the scale, codes within [-127, 127]
    codes = torch.round(y / 0.05)
    assert torch.equal(codes * 0.05, y) and float(codes.min()) >= -127 and float(codes.max()) <= 127
    # "+0.5f then truncate": error <= scale/2 for x >= 0, < 1.5 scale below
    err = (y - x).abs()
    assert err[x >= 0].max().item() <= 0.05 * 0.5 * 1.0001 and err.max().item() <= 0.05 * 1.5 * 1.0001
    rows = torch.randint(0, 64 * 1024, (96,), device="cuda")
    xs = x.view(-1, 1024)[rows].cpu().numpy()
    want = oracle.dequantize_linear(oracle.quantize_linear(xs, 0.05, 0, np.int8), 0.05, 0)
    np.testing.assert_array_equal(y.view(-1, 1024)[rows].cpu().numpy(), want)


def test_full_size_chain(g, oracle):
    """x, c [64,1024,1024], a, b [1024]: sampled rows against the oracle plus properties that do
    not depend on the size."""
    torch.manual_seed(1)
    x = torch.randn(64, 1024, 1024, device="cuda")
    c = torch.randn(64, 1024, 1024, device="cuda")
    a = torch.randn(1024, device="cuda")
    b = torch.randn(1024, device="cuda")
    y = g.ops.ElementWiseNvrtc([x, a, b, c], 1, chain_program(g.ops), 3)[0]
    torch.cuda.synchronize()
    assert y.shape == x.shape and float(y.min()) >= 0.0            # Relu
    assert bool(((y == 0) | (y > 0)).all())
    # |tanh * sigmoid| < 1, so y <= max(x + 1, 0)
    assert bool((y <= torch.clamp(x + 1, min=0)).all())
    rows = torch.randint(0, 64 * 1024, (96,), device="cuda")
    xs, cs = x.view(-1, 1024)[rows].cpu().numpy(), c.view(-1, 1024)[rows].cpu().numpy()
    want = oracle.run_chain(ORACLE_CHAIN, dict(x=xs, a=a.cpu().numpy(), b=b.cpu().numpy(), c=cs))["y"]
    np.testing.assert_array_equal(y.view(-1, 1024)[rows].cpu().numpy(), want)


def test_kernel_cache_and_errors(g):
    x = torch.randn(1000, device="cuda")
    prog = unary_program(g.ops, "Tanh")
    y1 = g.ops.ElementWiseNvrtc([x], 1, prog)[0]
    y2 = g.ops.ElementWiseNvrtc([x], 1, prog)[0]       # second call hits the cache
    torch.cuda.synchronize()
    assert torch.equal(y1, y2)
    with pytest.raises(g.capi.ChxHipError, match="fusable set"):
        g.ops.ElementWiseNvrtc([x], 1, unary_program(g.ops, "Erf"))
    with pytest.raises(g.capi.ChxHipError, match="does not broadcast"):
        g.ops.ElementWiseNvrtc([x, torch.randn(7, device="cuda")], 1,
                               g.ops.fusion_program([("x", F32), ("z", F32)], [("y", "Add", "x", "z")], [("y", F32)]),
                               outs=[torch.empty(1000, device="cuda")])


def test_random_programs(g, oracle):
    """Seeded random element-wise programs (every op of the generator, constants, operands that
    broadcast on inner and outer axes, one to three results) against the op-by-op CPU evaluation;
    bit-exact.  Exp only sees bounded values and divisors are positive, so no NaN arises whose
    ordering in Max / Min would be a matter of definition."""
    rng = np.random.default_rng(77)
    exact = {"Neg": np.negative, "Abs": np.abs, "Floor": np.floor, "Round": np.rint, "Max": np.maximum, "Min": np.minimum}
    shapes = [((4, 5, 33), (5, 1)), ((2, 3, 4, 129), (1, 129)), ((7, 64), (7, 1)), ((1000,), ()), ((3, 1, 17), (1, 6, 1)), ((2, 2, 2, 2, 5), (2, 1, 5))]
    for trial in range(24):
        shape, kshape = shapes[trial % len(shapes)]
        inputs = dict(x=(rng.standard_normal(shape) * 2).astype(np.float32), k=rng.standard_normal(kshape).astype(np.float32),
                      c=rng.standard_normal(shape).astype(np.float32))
        full_shape = np.broadcast_shapes(shape, kshape)
        stmts, pool, bounded = [], ["x", "k", "c"], set()
        shape_of = {n: v.shape for n, v in inputs.items()}

        def emit(op, *args):
            name = "v%d" % len(stmts)
            stmts.append((name, op) + args)
            pool.append(name)
            shape_of[name] = np.broadcast_shapes(*[shape_of[a] for a in args if isinstance(a, str)]) if op != "Const" else ()
            return name
        for _ in range(int(rng.integers(3, 14))):
            op = str(rng.choice(["Add", "Sub", "Mul", "Div", "Max", "Min", "Neg", "Abs", "Floor", "Round", "Relu", "Identity", "Tanh",
                                 "Sigmoid", "Exp", "Clip", "Const"]))
            a, b = (str(v) for v in rng.choice(pool, 2))
            if op == "Const":
                emit("Const", float(np.float32(rng.standard_normal())))
            elif op == "Clip":
                lo = float(np.float32(rng.uniform(-2, 0)))
                bounded.add(emit("Clip", a, lo, float(np.float32(lo + rng.uniform(0.1, 3)))))
            elif op in ("Tanh", "Sigmoid"):
                bounded.add(emit(op, a))
            elif op == "Exp":
                bounded.add(emit("Exp", a if a in bounded else emit("Tanh", a)))
            elif op == "Div":
                emit("Div", a, emit("Exp", emit("Tanh", b)))
            elif op in ("Add", "Sub", "Mul", "Max", "Min"):
                emit(op, a, b)
            else:
                emit(op, a)
        # results have the shape all operands broadcast to (runtime/ops/nvrtc.cc:100-113)
        candidates = [n for n in pool[3:] if tuple(shape_of[n]) == tuple(full_shape)]
        if not candidates:
            candidates = [emit("Add", emit("Add", pool[-1], "x"), "k")]
        outs = [str(n) for n in rng.choice(candidates, size=min(len(candidates), int(rng.integers(1, 4))), replace=False)]
        env = dict(inputs)
        for stmt in stmts:
            if stmt[1] in exact:
                env[stmt[0]] = exact[stmt[1]](*[env[a] for a in stmt[2:]]).astype(np.float32)
            else:
                env = oracle.run_chain([stmt], env)
        prog = g.ops.fusion_program([("x", F32), ("k", F32), ("c", F32)], stmts, [(o, F32) for o in outs])
        got = g.ops.ElementWiseNvrtc([g.dev(inputs[n]) for n in ("x", "k", "c")], len(outs), prog, 1000 + trial)
        for o, t in zip(outs, got):
            want = np.broadcast_to(env[o], full_shape)
            assert not np.isnan(want).any()
            np.testing.assert_array_equal(g.host(t), want, err_msg="trial %d, %s of %s" % (trial, o, stmts))


# ---- the CUDA C text of the reference's BuildNvrtcProgram (compiler/nvrtc_builder.cc:91-206) as the program ----

def _nvrtc_sources():
    import json
    import os
    with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "nvrtc_fusion_sources.json")) as f:
        return json.load(f)


def _chain_of_the_reference_text(orc, x, a, b, c, rnd):
    """The chain fixture operation by operation; `rnd` rounds every result to the program's type (identity for
    float32).  The sigmoid is that text's helper: tanh(x * 0.5) * 0.5 + 0.5."""
    half = rnd(np.float32(0.5))
    t0 = rnd(orc.binary(orc.MUL, x, a))
    s = rnd(orc.binary(orc.ADD, rnd(orc.binary(orc.MUL, rnd(orc.tanh(rnd(orc.binary(orc.MUL, c, half)))), half)), half))
    t1 = rnd(orc.binary(orc.ADD, t0, b))
    t2 = rnd(orc.tanh(t1))
    t4 = rnd(orc.binary(orc.MUL, t2, s))
    return rnd(orc.binary(orc.ADD, t4, x))


def test_reference_kernel_text_in_float(g, oracle):
    src = _nvrtc_sources()
    rng = np.random.default_rng(31)
    x = (rng.standard_normal((3, 40, 64)) * 2).astype(np.float32)
    got = g.host(g.ops.ElementWiseNvrtc([g.dev(x)], 1, src["tanh_sigmoid_float"], 1)[0])
    np.testing.assert_array_equal(got, oracle.sigmoid_tanh_form(oracle.tanh(x)))
    # how far that spelling of the sigmoid is from the CPU path's 1 / (1 + exp(-x)): reported by the oracle, a few ulp
    a, b = rng.standard_normal(64).astype(np.float32), rng.standard_normal(64).astype(np.float32)
    c = rng.standard_normal((3, 40, 64)).astype(np.float32)
    chain = src["chain_T"].replace("@T@", "float")
    got = g.host(g.ops.ElementWiseNvrtc([g.dev(x), g.dev(a), g.dev(b), g.dev(c)], 1, chain, 3)[0])
    np.testing.assert_array_equal(got, _chain_of_the_reference_text(oracle, x, a, b, c, lambda v: v))
    p, q = rng.standard_normal((7, 33)).astype(np.float32), rng.standard_normal((7, 33)).astype(np.float32)
    r, s = g.ops.ElementWiseNvrtc([g.dev(p), g.dev(q)], 2, src["const_sub_div_exp_identity_float"], 12)
    d = oracle.binary(oracle.SUB, p, q)
    want_r = oracle.binary(oracle.MUL, oracle.binary(oracle.DIV, oracle.exp(d), np.float32(2)), np.float32(0.333333))
    np.testing.assert_array_equal(g.host(r), want_r)
    np.testing.assert_array_equal(g.host(s), d)


def test_reference_kernel_text_in_half(g, oracle):
    """typedef half T: every node is a half-precision operation, i.e. the float32 operation rounded to float16
    (numpy's float16 arithmetic is defined the same way); tanh is the C library's float32 tanh, rounded."""
    rng = np.random.default_rng(32)
    h = lambda v: np.asarray(v, np.float32).astype(np.float16).astype(np.float32)
    x, c = h(rng.standard_normal((5, 24, 64)) * 2), h(rng.standard_normal((5, 24, 64)))
    a, b = h(rng.standard_normal(64)), h(rng.standard_normal(64))
    chain = _nvrtc_sources()["chain_T"].replace("@T@", "half")
    dev = [torch.from_numpy(v.astype(np.float16)).cuda() for v in (x, a, b, c)]
    got = g.ops.ElementWiseNvrtc(dev, 1, chain, 3)[0]
    assert got.dtype == torch.float16
    want = _chain_of_the_reference_text(oracle, x, a, b, c, h)
    np.testing.assert_array_equal(got.cpu().numpy(), want.astype(np.float16))
    # the exact operations, straight against numpy's float16 arithmetic
    xh, ah, bh = x.astype(np.float16), a.astype(np.float16), b.astype(np.float16)
    own = g.ops.fusion_program([("x", torch.float16), ("a", torch.float16), ("b", torch.float16)],
                               [("m", "Mul", "x", "a"), ("s", "Add", "m", "b"), ("d", "Div", "s", "a"), ("r", "Relu", "d")], [("r", torch.float16)])
    got = g.ops.ElementWiseNvrtc(dev[:3], 1, own, 4)[0].cpu().numpy()
    with np.errstate(all="ignore"):
        np.testing.assert_array_equal(got, np.maximum((xh * ah + bh) / ah, np.float16(0)))


def test_reference_kernel_text_in_double(g):
    """typedef double T: the arithmetic operations bit for bit against numpy's float64; tanh within 2 ulp of the C
    library's double-precision tanh (its bits are not pinned: the device's double tanh is the ROCm math library's)."""
    rng = np.random.default_rng(33)
    x, c = rng.standard_normal((5, 24, 64)) * 2, rng.standard_normal((5, 24, 64))
    a, b = rng.standard_normal(64), rng.standard_normal(64)
    own = g.ops.fusion_program([("x", torch.float64), ("a", torch.float64), ("b", torch.float64)],
                               [("m", "Mul", "x", "a"), ("s", "Add", "m", "b"), ("d", "Div", "s", "a"), ("u", "Sub", "d", "x"), ("r", "Relu", "u")],
                               [("r", torch.float64)])
    dev = [torch.from_numpy(v).cuda() for v in (x, a, b, c)]
    got = g.ops.ElementWiseNvrtc(dev[:3], 1, own, 5)[0]
    assert got.dtype == torch.float64
    np.testing.assert_array_equal(got.cpu().numpy(), np.maximum((x * a + b) / a - x, 0.0))
    chain = _nvrtc_sources()["chain_T"].replace("@T@", "double")
    got = g.ops.ElementWiseNvrtc(dev, 1, chain, 3)[0].cpu().numpy()
    want = np.tanh(x * a + b) * (np.tanh(c * 0.5) * 0.5 + 0.5) + x
    # two tanh results within 2 ulp each, carried through a product and two sums of magnitude <= 1 + |x|
    assert np.all(np.abs(got - want) <= 6 * np.spacing(1.0 + np.abs(x)))
    single = "typedef double T;\nextern \"C\" __global__\nvoid fusion9(size_t n, T* i_x, T* o_y) {\nconst T v_x = i_x[tid];\nconst T v_y = tanh(v_x);\no_y[tid] = v_y;\n}\n"
    got = g.ops.ElementWiseNvrtc(dev[:1], 1, single, 9)[0].cpu().numpy()
    assert np.all(np.abs(got - np.tanh(x)) <= 2 * np.spacing(np.abs(np.tanh(x))))
