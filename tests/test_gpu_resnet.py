"""Whole quantized networks on the MI355X against the CPU oracle executing the same
op program: every intermediate tensor must be bit-identical (uint8), the final
DequantizeLinear output identical as fp32."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def g():
    import gpu_util
    gpu_util.capi.init(0)
    return gpu_util


def check_model(g, oracle, model, threads=16):
    wl = g.pkg.workloads
    oracle.set_threads(threads)
    try:
        ref = wl.run_reference(model, oracle, model["input"])
    finally:
        oracle.set_threads(1)
    # every op a kernel of its own; then with the residual sums inside the convolutions before them (those
    # convolutions' own outputs are then not materialised); then also with the two convolutions that read a
    # down-sampling block's input as one launch
    for fuse, pair, signed in ((False, False, False), (True, False, False), (True, True, False), (True, True, True), (False, False, True)):
        runner = wl.DeviceRunner(model, g.pkg, fuse_residual=fuse, pair_convs=pair, minus_128=signed)
        dev = runner.run(torch.from_numpy(model["input"]).cuda())
        torch.cuda.synchronize()
        assert bool(runner.fused_into) == (fuse and any(i[0] in ("Add", "AddRelu") for i in model["program"]))
        paired = sum(1 for i in runner.program if i[0] == "QLinearConvPair")
        assert (paired > 0) == (pair and len(wl.pair_convolutions(model["program"], model["convs"])) < len(model["program"]))
        assert bool(runner.minus_128) == signed
        for ins in model["program"]:
            name = ins[1]
            if name in runner.fused_into:
                assert name not in dev
                continue
            got = dev[name]
            if name in runner.minus_128:
                # codes minus 128 in an int8 array: the values only convolutions read
                assert got.dtype == torch.int8
                got = got.view(torch.uint8) ^ 0x80
            np.testing.assert_array_equal(got.cpu().numpy(), ref[name],
                                          err_msg="value %s after %s (fused residual: %s, paired: %s, minus 128: %s)" % (name, ins[0], fuse, pair, signed))
        runner.close()
    return ref


def test_pooling_ops(g, oracle):
    rng = np.random.default_rng(41)
    x = rng.integers(0, 256, size=(2, 32, 13, 12)).astype(np.uint8)
    for cover_all in (False, True):
        want = oracle.max_pool_q8(x, (3, 3), (2, 2), (0, 0), cover_all)
        for xd in (g.dev(x), g.to_channels_last(g.dev(x))):
            np.testing.assert_array_equal(g.host(g.ops.MaxPoolQ8(xd, (3, 3), (2, 2), (0, 0), cover_all)), want)
    xi = rng.integers(-128, 128, size=(1, 16, 9, 9)).astype(np.int8)
    np.testing.assert_array_equal(g.host(g.ops.MaxPoolQ8(g.to_channels_last(g.dev(xi)), (2, 2), (2, 2), (1, 1))),
                                  oracle.max_pool_q8(xi, (2, 2), (2, 2), (1, 1)))
    # windows of more than nine taps (the kernel's load groups), one tap, padded on every side
    for k, st, pad in (((4, 5), (2, 3), (1, 2)), ((1, 1), (2, 2), (0, 0)), ((5, 5), (1, 1), (2, 2))):
        np.testing.assert_array_equal(g.host(g.ops.MaxPoolQ8(g.to_channels_last(g.dev(xi)), k, st, pad)),
                                      oracle.max_pool_q8(xi, k, st, pad), err_msg=str((k, st, pad)))
    want = oracle.average_pool_q8(x, 0.05, 30, (7, 7), (1, 1), (0, 0), 0.02, 7)
    np.testing.assert_array_equal(g.host(g.ops.AveragePoolQ8(g.to_channels_last(g.dev(x)), 0.05, 30, (7, 7), (1, 1), (0, 0),
                                                             0.02, 7)), want)
    assert want.min() < want.max()
    # max of the codes == Q(MaxPool(DQ(x))) spelled out on the CPU
    dq = oracle.dequantize_linear(x, 0.05, 30)
    pooled = np.stack([[dq[n, c, i:i + 3, j:j + 3].max() for i in range(0, 11, 2) for j in range(0, 10, 2)]
                       for n in range(2) for c in range(32)]).reshape(2, 32, 6, 5)
    np.testing.assert_array_equal(oracle.quantize_linear(pooled, 0.05, 30), oracle.max_pool_q8(x, (3, 3), (2, 2)))


@pytest.mark.parametrize("xdt", [np.uint8, np.int8])
@pytest.mark.parametrize("case", [
    # N, C, H, W, kernel, stride, pad, count_include_pad
    (2, 32, 7, 7, 7, 1, 0, False), (1, 20, 9, 11, 3, 2, 1, False), (1, 8, 6, 6, 3, 1, 1, True), (1, 12, 10, 13, 9, 1, 0, False),
    (2, 6, 5, 5, 2, 2, 0, False),
    # whole-image windows: 64 taps is the most the global-pool kernel takes, 81 goes the general way
    (1, 8, 8, 8, 8, 1, 0, False), (1, 8, 9, 9, 9, 1, 0, False), (3, 4, 1, 1, 1, 1, 0, False)])
def test_average_pool_layouts(g, oracle, case, xdt):
    """AveragePool between DequantizeLinear and QuantizeLinear: the four-channel channels-last
    kernel (also windows wider than its eight-tap groups, padding, both count modes, int8) and the
    generic one (NCHW operands, a channel count that is not a multiple of four) give the oracle's bytes."""
    N, C, H, W, k, s, pad, cip = case
    rng = np.random.default_rng(43)
    lo, hi = (0, 256) if xdt == np.uint8 else (-128, 128)
    x = rng.integers(lo, hi, size=(N, C, H, W)).astype(xdt)
    xz = 77 if xdt == np.uint8 else -12
    for ydt, yz, flags, rm in ((np.uint8, 9, 0, oracle.ROUND_REFERENCE), (np.int8, -30, g.capi.ROUND_ONNX_RNE, oracle.ROUND_ONNX_RNE)):
        want = oracle.average_pool_q8(x, 0.05, xz, (k, k), (s, s), (pad, pad), 0.031, yz, ydt, count_include_pad=cip, round_mode=rm)
        assert want.min() < want.max()
        zdt = torch.uint8 if ydt == np.uint8 else torch.int8
        for xd in (g.to_channels_last(g.dev(x)), g.dev(x)):
            got = g.ops.AveragePoolQ8(xd, 0.05, xz, (k, k), (s, s), (pad, pad), 0.031, yz, count_include_pad=cip,
                                      zero_point_dtype=zdt, flags=flags)
            np.testing.assert_array_equal(g.host(got), want)


def test_small_resnet_every_value(g, oracle):
    model = g.pkg.workloads.build_resnet50(batch=2, image=64, seed=5, width=16, blocks=(2, 1, 1, 1), classes=10)
    ref = check_model(g, oracle, model)
    # the quantized network tracks the float one it was calibrated on
    err = np.abs(ref["logits"].reshape(2, 10) - model["float_logits"].reshape(2, 10)).max()
    assert err < 0.25 * np.abs(model["float_logits"]).max() + 0.5


def test_resnet50_batch1(g, oracle):
    """The real architecture (ResNet-50 v1, 224x224) on one image."""
    model = g.pkg.workloads.build_resnet50(batch=1, seed=3)
    assert 3.8e9 < model["macs"] < 4.2e9
    check_model(g, oracle, model)


def test_hip_graph_replay_matches_eager(g, oracle):
    """The program captured into a HIP graph: several replays, with eager work and
    synchronizations in between, must each reproduce the eager result bit for bit."""
    wl = g.pkg.workloads
    model = wl.build_resnet50(batch=2, image=64, seed=6, width=16, blocks=(1, 1, 1, 1), classes=10)
    runner = wl.DeviceRunner(model, g.pkg)
    x = torch.from_numpy(model["input"]).cuda()
    eager = {k: v.clone() for k, v in runner.run(x).items()}
    torch.cuda.synchronize()
    replay = runner.capture(x)
    for i in range(4):
        for buf in runner.bufs.values():
            buf.zero_()                       # eager work between replays; also proves the replay recomputes
        torch.cuda.synchronize()
        out = replay()
        torch.cuda.synchronize()
        for ins in model["program"]:
            assert torch.equal(out[ins[1]], eager[ins[1]]), "replay %d: %s" % (i, ins[1])
    runner.close()


def test_small_mobilenetv2_every_value(g, oracle):
    """Reduced MobileNetV2: stem, inverted residual blocks with expansion, depthwise 3x3 at both
    strides, linear projections, residual Adds, head, pool, classifier."""
    blocks = ((1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 2, 2), (6, 64, 2, 1))
    model = g.pkg.workloads.build_mobilenetv2(batch=2, image=64, seed=7, blocks=blocks, stem=32, head=128, classes=10)
    kinds = [ins[0] for ins in model["program"]]
    assert "Add" in kinds and sum(c.group > 1 for c in model["convs"].values()) == 7
    ref = check_model(g, oracle, model)
    assert ref["logits_q"].min() < ref["logits_q"].max()


def test_mobilenetv2_batch1(g, oracle):
    """The real architecture (MobileNetV2-1.0, 224x224) on one image."""
    model = g.pkg.workloads.build_mobilenetv2(batch=1, seed=4)
    assert 2.9e8 < model["macs"] < 3.2e8          # ~300 MMAC per image
    assert sum(c.group > 1 for c in model["convs"].values()) == 17
    check_model(g, oracle, model)


def test_concurrent_batch_slices_match_whole_batch(g, oracle):
    """The batch run as concurrent slices on separate streams (eager and as a replayed HIP graph)
    gives the bytes of the whole-batch run."""
    wl = g.pkg.workloads
    model = wl.build_resnet50(batch=5, image=64, seed=8, width=16, blocks=(1, 1, 1, 1), classes=10)
    x = torch.from_numpy(model["input"]).cuda()
    whole = wl.DeviceRunner(model, g.pkg)
    want = {k: v.clone() for k, v in whole.run(x).items()}
    torch.cuda.synchronize()
    split = wl.ConcurrentRunner(model, g.pkg, parts=2)
    assert [hi - lo for lo, hi in split.slices] == [2, 3]

    def check(outs, tag):
        torch.cuda.synchronize()
        for ins in model["program"]:
            got = torch.cat([o[ins[1]] for o in outs], dim=0)
            assert torch.equal(got, want[ins[1]]), "%s: %s" % (tag, ins[1])
    check(split.run(x), "eager")
    replay = split.capture(x)
    for i in range(3):
        for r in split.runners:
            for buf in r.bufs.values():
                buf.zero_()
        torch.cuda.synchronize()
        check(replay(), "replay %d" % i)
    whole.close()
    split.close()


@pytest.mark.parametrize("net,batch,seed", [("resnet50", 64, 3), ("mobilenetv2", 128, 4)])
def test_benchmark_configuration_at_full_size(g, oracle, net, batch, seed):
    """The timed configuration itself: the full batch, residual sums inside the convolutions, the tuned
    launch configurations, one HIP graph replay.  Three images of the batch are followed through the
    oracle tensor by tensor; all of them through a property that needs no oracle: every op on the
    path is independent per image, so a permuted batch must give the permuted results."""
    wl = g.pkg.workloads
    model = (wl.build_resnet50 if net == "resnet50" else wl.build_mobilenetv2)(batch=batch, seed=seed)
    runner = wl.DeviceRunner(model, g.pkg, fuse_residual=True)
    assert runner.fused_into
    x = torch.from_numpy(model["input"]).cuda()
    runner.run(x)                      # eager first: the plans time their launch configurations here
    torch.cuda.synchronize()
    replay = runner.capture(x)
    out = {k: v.clone() for k, v in replay().items()}
    torch.cuda.synchronize()
    picks = [0, batch // 2 + 5, batch - 1]
    oracle.set_threads(16)
    try:
        ref = wl.run_reference(model, oracle, model["input"][picks])
    finally:
        oracle.set_threads(1)
    for ins in model["program"]:
        name = ins[1]
        if name in runner.fused_into:
            continue
        np.testing.assert_array_equal(out[name][picks].cpu().numpy(), ref[name], err_msg="%s after %s" % (name, ins[0]))
    perm = torch.randperm(batch, generator=torch.Generator().manual_seed(seed)).cuda()
    x.copy_(x[perm])
    again = replay()
    torch.cuda.synchronize()
    for name in ("logits_q", "logits"):
        assert torch.equal(again[name], out[name][perm]), name
    assert out["logits_q"].min() < out["logits_q"].max()
    runner.close()


def test_random_pool_sweep(g, oracle):
    """Seeded random MaxPool / AveragePool windows on quantized tensors: kernel, stride, pads,
    cover_all / count_include_pad, channel counts on and off the vector widths of the channels-last
    kernels, both layouts, both element types; bit-exact."""
    rng = np.random.default_rng(909)
    done = 0
    for trial in range(60):
        N, C = int(rng.integers(1, 4)), int(rng.choice([1, 3, 4, 8, 12, 16, 20, 32, 48, 64, int(rng.integers(1, 90))]))
        H, W = int(rng.integers(1, 20)), int(rng.integers(1, 20))
        kh, kw = int(rng.integers(1, 6)), int(rng.integers(1, 6))
        if trial % 6 == 0:
            kh, kw = H, W                                   # the window is the whole image
        sh, sw = int(rng.integers(1, 4)), int(rng.integers(1, 4))
        ph, pw = int(rng.integers(0, kh // 2 + 1)), int(rng.integers(0, kw // 2 + 1))
        if H + 2 * ph < kh or W + 2 * pw < kw:
            continue
        xdt = [np.uint8, np.int8][int(rng.integers(0, 2))]
        lo, hi = (0, 256) if xdt == np.uint8 else (-128, 128)
        x = rng.integers(lo, hi, size=(N, C, H, W)).astype(xdt)
        xd = g.dev(x) if rng.integers(0, 3) == 0 else g.to_channels_last(g.dev(x))
        tag = "trial %d: x%s %s kernel %s strides %s pads %s" % (trial, x.shape, xdt.__name__, (kh, kw), (sh, sw), (ph, pw))
        cover_all = bool(rng.integers(0, 2))
        np.testing.assert_array_equal(g.host(g.ops.MaxPoolQ8(xd, (kh, kw), (sh, sw), (ph, pw), cover_all)),
                                      oracle.max_pool_q8(x, (kh, kw), (sh, sw), (ph, pw), cover_all), err_msg=tag + " max, cover_all %s" % cover_all)
        cip = bool(rng.integers(0, 2))
        xz = int(rng.integers(lo, hi))
        ydt = [np.uint8, np.int8][int(rng.integers(0, 2))]
        yz = int(rng.integers(0, 256) if ydt == np.uint8 else rng.integers(-128, 128))
        ys = np.float32(rng.uniform(0.02, 0.08))
        want = oracle.average_pool_q8(x, 0.05, xz, (kh, kw), (sh, sw), (ph, pw), ys, yz, ydt, count_include_pad=cip)
        got = g.ops.AveragePoolQ8(xd, 0.05, xz, (kh, kw), (sh, sw), (ph, pw), ys, yz, count_include_pad=cip,
                                  zero_point_dtype=torch.uint8 if ydt == np.uint8 else torch.int8)
        np.testing.assert_array_equal(g.host(got), want, err_msg=tag + " average, count_include_pad %s -> %s" % (cip, ydt.__name__))
        done += 1
    assert done >= 50
