"""QuantizeLinear / DequantizeLinear on the MI355X through the C ABI, bit-exact
against the CPU oracle (runtime/ops/quantize.cc:16-60 restated)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def g():
    import gpu_util
    gpu_util.capi.init(0)
    return gpu_util


CASES = [(np.uint8, 128, 0.02), (np.uint8, 0, 1.0 / 255), (np.int8, 0, 0.05), (np.int8, -7, 0.3),
         (np.uint8, 255, 3.0), (np.uint8, 128, 2.0)]


@pytest.mark.parametrize("dtype,zp,scale", CASES)
@pytest.mark.parametrize("n", [1, 15, 16, 17, 4099, 1 << 20])
def test_quantize_matches_oracle(g, oracle, dtype, zp, scale, n):
    rng = np.random.default_rng(n)
    x = (rng.standard_normal(n) * 20 * scale * 8).astype(np.float32)
    k = min(n, 600)
    x[:k] = ((np.arange(k) - k // 2) + 0.5).astype(np.float32) * np.float32(scale)  # exact .5 ties
    tdt = torch.uint8 if dtype == np.uint8 else torch.int8
    for flags, mode in ((0, oracle.ROUND_REFERENCE), (g.capi.ROUND_ONNX_RNE, oracle.ROUND_ONNX_RNE)):
        y = g.host(g.ops.QuantizeLinear(g.dev(x), scale, zp, tdt, flags=flags))
        assert y.dtype == dtype
        np.testing.assert_array_equal(y, oracle.quantize_linear(x, scale, zp, dtype, round_mode=mode))


def test_quantize_onnx_vector(g, onnx_vectors):
    t = onnx_vectors["test_quantizelinear"]
    y = g.host(g.ops.QuantizeLinear(g.dev(np.array(t["x"], np.float32)), t["y_scale"], t["y_zero_point"], torch.uint8))
    assert y.tolist() == t["y"]


def test_dequantize_onnx_vector(g, onnx_vectors):
    t = onnx_vectors["test_dequantizelinear"]
    y = g.host(g.ops.DequantizeLinear(g.dev(np.array(t["x"], np.uint8)), t["x_scale"], t["x_zero_point"]))
    assert y.dtype == np.float32 and y.tolist() == t["y"]


@pytest.mark.parametrize("dtype,zp,scale", CASES)
@pytest.mark.parametrize("n", [1, 31, 4096 + 5, 1 << 20])
def test_dequantize_matches_oracle(g, oracle, dtype, zp, scale, n):
    rng = np.random.default_rng(n + 1)
    lo, hi = (0, 256) if dtype == np.uint8 else (-128, 128)
    q = rng.integers(lo, hi, size=n).astype(dtype)
    y = g.host(g.ops.DequantizeLinear(g.dev(q), scale, zp))
    np.testing.assert_array_equal(y, oracle.dequantize_linear(q, scale, zp))


def test_default_zero_point_is_uint8_zero(g, oracle):
    x = np.linspace(-3, 300, 1000).astype(np.float32)
    y = g.host(g.ops.QuantizeLinear(g.dev(x), 1.0))
    assert y.dtype == np.uint8
    np.testing.assert_array_equal(y, oracle.quantize_linear(x, 1.0, 0, np.uint8))


def test_strided_and_channels_last_views(g, oracle):
    rng = np.random.default_rng(5)
    x = rng.standard_normal((3, 5, 6, 7)).astype(np.float32) * 4
    want = oracle.quantize_linear(x, 0.05, 128, np.uint8)
    xd = g.dev(x)
    # channels-last input and output views: flat walk over identical dense layouts
    y = g.ops.QuantizeLinear(g.to_channels_last(xd), 0.05, 128, torch.uint8)
    assert y.stride() == g.to_channels_last(xd).stride()
    np.testing.assert_array_equal(g.host(y), want)
    # NCHW input, channels-last output: generic strided kernel
    out = torch.empty((3, 6, 7, 5), dtype=torch.uint8, device="cuda").permute(0, 3, 1, 2)
    g.ops.QuantizeLinear(xd, 0.05, 128, torch.uint8, out=out)
    np.testing.assert_array_equal(g.host(out), want)
    # sliced (gappy) input
    big = g.dev(rng.standard_normal((4, 10, 12)).astype(np.float32))
    view = big[:, 2:9:2, 1:11]
    out2 = torch.empty(view.shape, dtype=torch.int8, device="cuda")
    g.ops.QuantizeLinear(view, 0.1, -3, torch.int8, out=out2)
    np.testing.assert_array_equal(g.host(out2), oracle.quantize_linear(g.host(view), 0.1, -3, np.int8))
    # dequantize back through a strided output
    dq = torch.empty((3, 6, 7, 5), dtype=torch.float32, device="cuda").permute(0, 3, 1, 2)
    g.ops.DequantizeLinear(g.dev(want), 0.05, 128, out=dq)
    np.testing.assert_array_equal(g.host(dq), oracle.dequantize_linear(want, 0.05, 128))


def test_full_size_round_trip_properties(g, oracle):
    """[64,1024,1024] fp32 (the element-wise configuration's x): checked through
    size-independent properties and a sampled comparison with the oracle."""
    torch.manual_seed(1)
    x = torch.randn(64, 1024, 1024, device="cuda")
    q = g.ops.QuantizeLinear(x, 0.05, 0, torch.int8)
    d = g.ops.DequantizeLinear(q, 0.05, 0)
    q2 = g.ops.QuantizeLinear(d, 0.05, 0, torch.int8)
    torch.cuda.synchronize()
    # Q(DQ(q)) == q for q >= 0; for q < 0 the reference's "+0.5f then truncate" lands on q + 1
    assert torch.equal(q2, torch.where(q < 0, q + 1, q))
    assert int(q.min()) >= -127 and int(q.max()) <= 127
    # "+0.5f then truncate" is round-half-up for x >= 0 (error <= scale/2) and truncation of
    # x/scale + 0.5 toward zero for x < 0 (error < 1.5 scale)
    err = (d - x).abs()
    assert err[x >= 0].max().item() <= 0.05 * 0.5 * 1.0001
    assert err.max().item() <= 0.05 * 1.5 * 1.0001
    u = g.ops.QuantizeLinear(x, 0.05, 128, torch.uint8)
    assert torch.equal(g.ops.QuantizeLinear(g.ops.DequantizeLinear(u, 0.05, 128), 0.05, 128, torch.uint8), u)
    idx = torch.randint(0, 64 * 1024 * 1024 // 4096, (257,), device="cuda")
    rows = x.view(-1, 4096)[idx]
    np.testing.assert_array_equal(q.view(-1, 4096)[idx].cpu().numpy(),
                                  oracle.quantize_linear(rows.cpu().numpy(), 0.05, 0, np.int8))


def test_errors(g):
    x = torch.zeros(8, device="cuda")
    with pytest.raises(g.capi.ChxHipError, match="zero point"):
        g.ops.QuantizeLinear(x, 1.0, 300, torch.uint8)
    with pytest.raises(g.capi.ChxHipError, match="float32"):
        g.ops.QuantizeLinear(x.to(torch.float64), 1.0, 0, torch.uint8)
    with pytest.raises(g.capi.ChxHipError, match="shapes differ"):
        g.ops.QuantizeLinear(x, 1.0, 0, torch.uint8, out=torch.empty(9, dtype=torch.uint8, device="cuda"))
    # empty input is fine
    assert g.ops.QuantizeLinear(torch.zeros(0, device="cuda"), 1.0).numel() == 0


def test_bit_shift_against_numpy(g, vm=None):
    """BitShiftOp (runtime/ops/quantize.cc:153-163): both directions, every integer type of the array library, with
    broadcasting; counts below the element width, where numpy, C and the ONNX operator agree, plus numpy's results
    for counts of the width and beyond."""
    rng = np.random.default_rng(51)
    for dt, lo, hi in ((np.uint8, 0, 256), (np.int8, -128, 128), (np.int16, -2 ** 15, 2 ** 15), (np.int32, -2 ** 31, 2 ** 31),
                       (np.int64, -2 ** 62, 2 ** 62)):
        bits = np.dtype(dt).itemsize * 8
        x = rng.integers(lo, hi, size=(3, 5, 17)).astype(dt)
        y = rng.integers(0, bits, size=(5, 1)).astype(dt)
        for direction, fn in (("LEFT", np.left_shift), ("RIGHT", np.right_shift)):
            got = g.ops.BitShift(g.dev(x), g.dev(y), direction)
            assert tuple(got.shape) == (3, 5, 17)
            np.testing.assert_array_equal(g.host(got), fn(x, y), err_msg="%s %s" % (np.dtype(dt).name, direction))
            # a strided operand, and counts from the width upwards
            big = np.array([bits, bits + 3, 100 if bits > 8 else 77], dt)
            got = g.ops.BitShift(g.dev(x).permute(2, 0, 1)[:3], g.dev(big).reshape(3, 1, 1), direction)
            want = np.where(np.transpose(x, (2, 0, 1))[:3] < 0, -1, 0).astype(dt) if direction == "RIGHT" else np.zeros((3, 3, 5), dt)
            np.testing.assert_array_equal(g.host(got), want)
    # the ONNX operator's own examples (uint8)
    x, y = np.array([16, 4, 1], np.uint8), np.array([1, 2, 3], np.uint8)
    assert g.host(g.ops.BitShift(g.dev(x), g.dev(y), "RIGHT")).tolist() == [8, 1, 0]
    assert g.host(g.ops.BitShift(g.dev(x), g.dev(y), "LEFT")).tolist() == [32, 16, 8]
    with pytest.raises(g.capi.ChxHipError):
        g.ops.BitShift(g.dev(np.zeros(3, np.float32)), g.dev(np.zeros(3, np.float32)), "LEFT")
