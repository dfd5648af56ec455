#!/usr/bin/env python3
"""Benchmark of the quantized-inference path on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload resnet50|mobilenetv2|conv3x3|fusion|qdq]

Default workload: ResNet-50 v1 int8 QDQ inference, batch 64, 224x224 (the configuration the
headline metric is quoted on).  One step = one pass of the whole op program over one batch
that is already resident in HBM (fp32 NCHW input; QuantizeLinear is part of the step).
Prints ONE JSON line.  `roofline` describes the dominant kernel (the int8 MFMA implicit-GEMM
convolution for resnet50 / conv3x3, the fused element-wise kernel for fusion / qdq), timed
live with events on the launch stream: around every launch of the timed region for the
single-kernel workloads; for the networks (whose timed region is a HIP graph replay, where
no events can be placed) the convolution launches of the step are recorded in program order
into a graph of their own, which is replayed ten times between one event pair right after
the timed region.  `cpu_baseline` times the
restated reference CPU op sequence (the oracle's literal fp32 path) on the host cores for a
bounded sample of the same workload.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

INT8_PEAK_TOPS = 5000.0   # MI355X dense int8, published
HBM_PEAK_GBS = 8000.0     # MI355X HBM3E, published


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="resnet50", choices=["resnet50", "mobilenetv2", "conv3x3", "fusion", "qdq"])
    ap.add_argument("--batch", type=int, default=0, help="override the batch size (changes the workload; for experiments)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-graph", action="store_true", help="launch every op from the host instead of replaying a HIP graph")
    ap.add_argument("--cpu-seconds", type=float, default=20.0, help="rough budget for the CPU baseline")
    ap.add_argument("--no-fuse-residual", action="store_true",
                    help="run the residual Add(+Relu) groups as kernels of their own instead of inside the convolution before them")
    ap.add_argument("--no-pair-convs", action="store_true",
                    help="run the two convolutions that read a down-sampling block's input as two launches instead of one")
    ap.add_argument("--no-minus-128", action="store_true",
                    help="keep every 8-bit value between two convolutions as uint8 codes instead of codes minus 128 in int8 arrays")
    ap.add_argument("--parts", type=int, default=1,
                    help="run the batch as this many concurrent slices on separate streams (network workloads)")
    ap.add_argument("--runner", default="chxvm", choices=["chxvm", "python"],
                    help="network workloads: chxvm = the serialized ChxVMProgramProto through the C++ VM of the runtime library "
                         "(libchxvm_hip_runtime.so), its run recorded into a device graph and replayed; python = the op program "
                         "driven from Python through the C ABI (ops.py), also replayed as a graph")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="default workload only: do not append the short runs of the other configurations (other_workloads)")
    ap.add_argument("--copy-probe-mib", type=int, default=0,
                    help="also run one plain copy kernel (fused Identity on float32) over this many MiB: the known traffic "
                         "that hardware counters of a profiling run are scaled against")
    return ap.parse_args()


def timed_steps(torch, step, steps, warmup, instrument=None):
    """W untimed steps, then exactly K timed steps between two synchronizations."""
    for _ in range(warmup):
        step(None)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step(instrument)
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


class KernelTimer(object):
    """Event pairs around chosen launches on the current (launch) stream."""

    def __init__(self, torch):
        self.torch = torch
        self.pairs = []

    def wrap(self, tag, fn):
        a = self.torch.cuda.Event(enable_timing=True)
        b = self.torch.cuda.Event(enable_timing=True)
        a.record()
        r = fn()
        b.record()
        self.pairs.append((tag, a, b))
        return r

    def totals(self):
        out = {}
        for tag, a, b in self.pairs:
            ms = a.elapsed_time(b)
            cnt, tot = out.get(tag, (0, 0.0))
            out[tag] = (cnt + 1, tot + ms)
        return out


def cpu_info():
    model = "unknown"
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    return model, os.cpu_count() or 1


# ------------------------------------------------------------------------------------------------

def bench_resnet50(args, torch, pkg, mobilenet=False):
    wl = pkg.workloads
    batch = args.batch or (128 if mobilenet else 64)
    build = (lambda **kw: wl.build_mobilenetv2(seed=4, **kw)) if mobilenet else (lambda **kw: wl.build_resnet50(seed=3, **kw))
    model = build(batch=batch)
    x = torch.from_numpy(model["input"]).cuda()
    ops, capi = pkg.ops, pkg.capi
    conv_ops = 2.0 * model["macs"]

    # --parts N runs the batch as N concurrent slices on separate streams (the values are those of
    # the whole-batch run; a single ResNet layer at batch 64 is too few work-groups to keep 256
    # compute units busy through its ramp and tail, so slices fill each other's gaps).  The
    # default is the plain whole-batch runner, whose launches are the ones the roofline figure
    # below prices.
    fuse = not args.no_fuse_residual
    pair = fuse and not args.no_pair_convs and args.parts <= 1
    signed = fuse and not args.no_minus_128 and args.parts <= 1
    # values share memory once their last reader has run, as in the VM (whose allocator reuses freed slots)
    runner = wl.DeviceRunner(model, pkg, fuse, reuse_buffers=True, pair_convs=pair, minus_128=signed) if args.parts <= 1 else None
    timed_runner = runner if args.parts <= 1 else wl.ConcurrentRunner(model, pkg, args.parts, fuse)

    def step(_timer):
        timed_runner.run(x)

    # The timed region replays the whole program as one HIP graph (about 125 launches per step
    # would otherwise be bound by the host); --no-graph launches every op from the host instead.
    vm_prog = vm_replay = None
    use_vm = args.runner == "chxvm" and args.parts <= 1 and fuse
    if use_vm:
        # the drop-in itself: the network as one serialized program in the C++ VM
        import importlib
        vm = importlib.import_module(pkg.__name__ + ".chxvm")
        vm.set_option("pair_convolutions", "on" if pair else "off")
        vm.set_option("store_minus_128", "on" if signed else "off")
        vm_prog = vm.Program(wl.program_to_chxvm(model, vm, ops, keep=("logits",)).serialize())
        vm_prog.set_option("qlinearconv_bias", "onnx_int32")
        if args.no_graph:
            def step(_timer):  # noqa: F811  (the host walks the instructions; results are copied back, as run_onnx does)
                vm_prog.run({"x": x})
            sec = timed_steps(torch, step, args.steps, args.warmup)
        else:
            vm_replay = vm_prog.capture({"x": x})
            stream = capi.stream_ptr()
            sec = timed_steps(torch, lambda _t: vm_replay.launch(stream), args.steps, args.warmup)
    elif args.no_graph:
        sec = timed_steps(torch, step, args.steps, args.warmup)
    else:
        replay = timed_runner.capture(x)
        sec = timed_steps(torch, lambda _t: replay(), args.steps, args.warmup)

    # Launch duration of the dominant kernel: event pairs cannot be recorded inside a graph
    # replay, and around single 10-60 us launches they mostly measure submission gaps.  So the
    # QLinearConv instructions of the program (for MobileNetV2: the depthwise ones) are recorded,
    # in program order and on the buffers of the step just timed, into a graph of their own;
    # that graph is replayed REP times between one event pair on the launch stream.  Every layer
    # then finds its input where the timed step leaves it (written many launches earlier, not
    # just re-read), and launches follow each other without host submission gaps.
    REP = 10
    # the launches timed are those of the timed region: one slice's instructions, times the slices
    slices = [(runner, x)] if args.parts <= 1 else [(r, x[lo:hi]) for (lo, hi), r in zip(timed_runner.slices, timed_runner.runners)]
    conv_ms_per_step, n_launch = 0.0, 0
    layer_graphs = []
    for rn, xs in slices:
        rn.run(xs)
        torch.cuda.synchronize()
        vals = dict(rn.bufs, x=xs)   # every value's buffer (with reuse_buffers several share memory, as in the timed step)
        fids = []
        for fid, ins in enumerate(rn.program):
            if ins[0] not in ("QLinearConv", "QLinearConvPair"):
                continue
            if mobilenet and model["convs"][ins[3]].group == 1:
                continue  # MobileNetV2: the roofline figure is the depthwise kernel's
            fids.append(fid)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for fid in fids:
                rn.launch(fid, vals)   # as the timed step launches it (with its residual sum when that is fused in)
        layer_graphs.append(g)
        g.replay()
        a = torch.cuda.Event(enable_timing=True)
        b = torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(REP):
            g.replay()
        b.record()
        torch.cuda.synchronize()
        conv_ms_per_step += a.elapsed_time(b) / REP
        n_launch += len(fids)
    # What the event figure contains besides the kernels: in a graph every kernel boundary costs a fixed time
    # (the device hands one kernel's results to the next).  The same number of launches of a kernel that does
    # nothing, timed the same way, measures it; a profiler's per-kernel durations leave most of it out, so the
    # figure without it is the one to hold against profiles/.  frac below keeps the boundaries in.
    tiny = torch.zeros(64, device="cuda")
    idle = torch.cuda.CUDAGraph()
    with torch.cuda.graph(idle):
        for _ in range(n_launch):
            tiny.add_(1.0)
    idle.replay()
    a = torch.cuda.Event(enable_timing=True)
    b = torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(REP):
        idle.replay()
    b.record()
    torch.cuda.synchronize()
    boundary_ms_per_step = a.elapsed_time(b) / REP
    layer_graphs.append(idle)
    if mobilenet:
        achieved = model["depthwise_bytes"] / (conv_ms_per_step * 1e-3) / 1e9
        roofline = dict(bound="hbm", kernel="depthwise3x3_kernel (%d launches per step, summed)" % n_launch,
                        achieved=achieved, peak=HBM_PEAK_GBS, unit="GB/s", frac=achieved / HBM_PEAK_GBS, traffic=None,
                        bytes_per_step=model["depthwise_bytes"], kernel_ms_per_step=conv_ms_per_step)
    else:
        achieved = conv_ops / (conv_ms_per_step * 1e-3) / 1e12
        roofline = dict(bound="mfma", kernel="QLinearConv launches of one step, summed (%d: conv_mfma_kernel, the first layer conv_stem_kernel)" % n_launch,
                        achieved=achieved, peak=INT8_PEAK_TOPS, unit="TOP/s", frac=achieved / INT8_PEAK_TOPS, traffic=None,
                        ops_per_step=conv_ops, kernel_ms_per_step=conv_ms_per_step)
    # The same launches against BOTH roofs: a launch is priced at the roof that takes longer for its algorithmic
    # operations and bytes (input pixels it needs, weights, output, residual operand; workloads.conv_layer_table);
    # most 1x1 layers of these networks are below the ridge of 625 op/byte and belong to the HBM roof.  For
    # MobileNetV2 the figure covers every QLinearConv launch, not only the depthwise ones timed above.
    table = wl.conv_layer_table(model, fuse, pair)
    floor_s = sum(max(r["ops"] / (INT8_PEAK_TOPS * 1e12), r["bytes"] / (HBM_PEAK_GBS * 1e9)) for r in table)
    n_mfma = sum(1 for r in table if r["ops"] / (INT8_PEAK_TOPS * 1e12) >= r["bytes"] / (HBM_PEAK_GBS * 1e9))
    roofline["mixed"] = dict(
        floor_ms=floor_s * 1e3, mfma_only_ms=sum(r["ops"] for r in table) / (INT8_PEAK_TOPS * 1e12) * 1e3,
        hbm_only_ms=sum(r["bytes"] for r in table) / (HBM_PEAK_GBS * 1e9) * 1e3,
        algorithmic_bytes_per_step=sum(r["bytes"] for r in table), launches=len(table),
        launches_mfma_class=n_mfma, launches_hbm_class=len(table) - n_mfma)
    if not mobilenet:
        roofline["mixed"]["frac"] = floor_s * 1e3 / conv_ms_per_step
    roofline["launches_per_step"] = len(model["program"]) - (sum(1 for r in table if r["residual"]) if fuse else 0) - (
        len(wl.conv_layer_table(model, fuse)) - len(table))
    roofline["paired_convolutions"] = len(wl.conv_layer_table(model, fuse)) - len(table)
    roofline["boundary_us_per_launch"] = boundary_ms_per_step * 1e3 / max(n_launch, 1)
    roofline["kernel_ms_per_step_without_boundaries"] = conv_ms_per_step - boundary_ms_per_step
    roofline["frac_without_boundaries"] = roofline["frac"] * conv_ms_per_step / max(conv_ms_per_step - boundary_ms_per_step, 1e-9)
    if not mobilenet and batch == 64 and args.parts <= 1:
        # HBM bytes of the same launches from hardware counters (FETCH_SIZE / WRITE_SIZE, scaled by a
        # copy kernel of known size): NOT measured in this run but taken from two separate profiling runs,
        # kept with their commands; traffic_source says which file, so a reader can see how old it is
        try:
            t = json.load(open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "profiles",
                                            "resnet50_bs64_conv_mfma_traffic.json")))
            roofline["traffic"] = t["bytes_per_step"]
            roofline["traffic_source"] = "profiles/resnet50_bs64_conv_mfma_traffic.json (%s)" % t.get("measured_at", "separate rocprofv3 --pmc runs")
        except (OSError, ValueError, KeyError):
            pass
    # the launch configurations the plans measured for these launches: tile (output channels x pixels),
    # work-groups per compute unit (0 = as many as fit) and wavefronts per work-group -> number of layers
    hist, forms = {}, {}
    for rn, _xs in slices:
        for plan in rn.plans.values():
            for line in plan.describe():
                f = dict(kv.split("=") for kv in line.split() if "=" in kv)
                if "residual" in f:
                    # the fused residual sum of this layer: two multiply-adds with constants that the plan's search
                    # found exact on all code pairs ("affine"), or the operation-by-operation arithmetic ("exact")
                    forms[f["residual"]] = forms.get(f["residual"], 0) + 1
                    continue
                key = "%s/%s/w%s%s" % (f.get("tile"), f.get("wgs_per_cu"), f.get("waves", "4"), "+res" if f.get("res") == "1" else "")
                hist[key] = hist.get(key, 0) + 1
    roofline["configs"] = hist
    roofline["configs_source"] = ("plans of the Python runner (ops.py), whose launches the kernel time above is measured on; the "
                                  "plans inside the C++ VM measure their own configurations and may choose differently")
    if forms:
        roofline["residual_sums"] = forms
    res = dict(metric="images/sec %s int8 bs%d @1 GPU" % ("MobileNetV2" if mobilenet else "ResNet-50", batch),
               value=batch / sec, unit="images/sec", ms_per_step=sec * 1e3, dtype="int8",
               config=dict(workload="mobilenetv2_int8_qdq" if mobilenet else "resnet50_v1_int8_qdq", batch=batch, image=224,
                           layout="channels_last", launch="host" if args.no_graph else "hip_graph_replay",
                           runner="chxvm (serialized ChxVMProgramProto in libchxvm_hip_runtime.so)" if use_vm else "python (ops.py over the C ABI)",
                           concurrent_batch_slices=max(1, args.parts), residual_add="separate" if args.no_fuse_residual else "in_conv_epilogue",
                           conv_gmac_per_image=model["macs"] / batch / 1e9))

    def cpu():
        from oracle import oracle as orc
        lit = _literal_executor(orc)
        cores = orc.max_threads()
        one = build(batch=1)
        orc.set_threads(1)
        t0 = time.perf_counter()
        wl.run_reference(one, lit, one["input"])
        dt1 = time.perf_counter() - t0
        # all cores, sized to roughly the requested budget
        nb = int(max(1, min(batch, args.cpu_seconds / max(dt1 / cores * 1.5, 1e-3))))
        many = model if nb == batch else build(batch=nb)
        orc.set_threads(cores)
        t0 = time.perf_counter()
        wl.run_reference(many, lit, many["input"])
        dtn = time.perf_counter() - t0
        # Where the integer-accumulating restatement (which the device is held to, bit for bit) and the literal fp32
        # restatement of QLinearConvOp differ: every convolution of three images computed both ways on the same
        # input.  Reported, not gated.
        three = build(batch=3)
        cnt = _MismatchCounter(orc)
        wl.run_reference(three, cnt, three["input"])
        orc.set_threads(1)
        parity = dict(images=3, elements=cnt.elements, literal_differs_from_int=cnt.differ,
                      largest_difference_in_codes=cnt.largest, layers_with_a_difference=cnt.layers)
        return dict(value=nb / dtn, unit="images/sec", cores=cores, kind="port", single_thread_value=1.0 / dt1, literal_vs_int=parity,
                    sample="%d images of the same network (batch %d), restated reference op sequence (fp32 dequantize, "
                           "im2col + sequential-k fp32 GEMM, quantize) with OpenMP over %d threads: %.1f s; one image "
                           "single-threaded, as ChainerX's native device runs: %.1f s" % (nb, nb, cores, dtn, dt1))
    def runner_close():
        if vm_replay is not None:
            vm_replay.close()
        if vm_prog is not None:
            vm_prog.close()
        timed_runner.close()
    return res, roofline, cpu, runner_close


def _literal_executor(orc):
    """The oracle with QLinearConv routed to the literal fp32 restatement of the reference."""
    class Lit(object):
        def __getattr__(self, name):
            return getattr(orc, name)

        def qlinear_conv_int(self, *a, **k):
            return orc.qlinear_conv_literal(*a, **k)
    return Lit()


class _MismatchCounter(object):
    """The oracle with QLinearConv computed both ways: returns the integer-accumulating result, counts the output
    elements on which the literal fp32 restatement differs from it."""

    def __init__(self, orc):
        self.orc, self.elements, self.differ, self.largest, self.layers = orc, 0, 0, 0, 0

    def __getattr__(self, name):
        return getattr(self.orc, name)

    def qlinear_conv_int(self, *a, **k):
        import numpy as np
        yi = self.orc.qlinear_conv_int(*a, **k)
        yl = self.orc.qlinear_conv_literal(*a, **k)
        d = np.abs(yi.astype(np.int32) - yl.astype(np.int32))
        self.elements += d.size
        self.differ += int(np.count_nonzero(d))
        self.largest = max(self.largest, int(d.max()) if d.size else 0)
        self.layers += 1 if d.any() else 0
        return yi


def bench_conv3x3(args, torch, pkg):
    import numpy as np
    ops, capi = pkg.ops, pkg.capi
    n = args.batch or 32
    rng = np.random.default_rng(2)
    x = rng.integers(0, 256, size=(n, 128, 28, 28)).astype(np.uint8)
    w = rng.integers(-127, 128, size=(128, 128, 3, 3)).astype(np.int8)
    ws = rng.uniform(0.001, 0.01, size=128).astype(np.float32)
    wz = np.zeros(128, np.int8)
    bias = rng.integers(-1000, 1001, size=128).astype(np.int32)
    xd = torch.from_numpy(x).cuda().permute(0, 2, 3, 1).contiguous().permute(0, 3, 1, 2)
    plan = ops.QLinearConvPlan(*[torch.from_numpy(a).cuda() for a in (w, ws, wz, bias)], pads=(1, 1))
    y = plan.run(xd, 0.02, 128, 0.05, 128, flags=capi.BIAS_ONNX_INT32)
    mac = n * 28 * 28 * 128 * 128 * 9

    fn = lambda: plan.run(xd, 0.02, 128, 0.05, 128, flags=capi.BIAS_ONNX_INT32, out=y)

    def step(_timer):
        fn()

    sec = timed_steps(torch, step, args.steps, args.warmup)
    # Launch duration: one event pair around K more launches, queued behind a sleeping kernel so
    # that the GPU runs them back to back (a pair around one 16 us launch measures submission).
    torch.cuda._sleep(int(2.4e9 * 0.002))
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ev0.record()
    for _ in range(args.steps):
        fn()
    ev1.record()
    torch.cuda.synchronize()
    ms, cnt = ev0.elapsed_time(ev1), args.steps
    achieved = 2.0 * mac / (ms / cnt * 1e-3) / 1e12
    roofline = dict(bound="mfma", kernel="conv_mfma_kernel", achieved=achieved, peak=INT8_PEAK_TOPS, unit="TOP/s",
                    frac=achieved / INT8_PEAK_TOPS, traffic=None, ops_per_launch=2.0 * mac, launch_us=ms / cnt * 1e3)
    res = dict(metric="images/sec QLinearConv 3x3 128->128 @28x28 (ResNet-50 stage 3), 1 GPU", value=n / sec,
               unit="images/sec", ms_per_step=sec * 1e3, dtype="int8",
               config=dict(workload="qlinearconv_3x3_c128_28x28", batch=n, layout="channels_last"))

    def cpu():
        from oracle import oracle as orc
        cores = orc.max_threads()
        orc.set_threads(cores)
        reps = 30
        t0 = time.perf_counter()
        for _ in range(reps):
            orc.qlinear_conv_literal(x, 0.02, 128, w, ws, wz, 0.05, 128, np.uint8, bias=bias, pads=(1, 1),
                                     bias_mode=orc.BIAS_ONNX_INT32)
        dt = time.perf_counter() - t0
        orc.set_threads(1)
        t1 = time.perf_counter()
        orc.qlinear_conv_literal(x, 0.02, 128, w, ws, wz, 0.05, 128, np.uint8, bias=bias, pads=(1, 1),
                                 bias_mode=orc.BIAS_ONNX_INT32)
        dt1 = time.perf_counter() - t1
        orc.set_threads(cores)
        cnt = _MismatchCounter(orc)
        cnt.qlinear_conv_int(x, 0.02, 128, w, ws, wz, 0.05, 128, np.uint8, bias=bias, pads=(1, 1), bias_mode=orc.BIAS_ONNX_INT32)
        orc.set_threads(1)
        parity = dict(elements=cnt.elements, literal_differs_from_int=cnt.differ, largest_difference_in_codes=cnt.largest)
        return dict(value=reps * n / dt, unit="images/sec", cores=cores, kind="port", single_thread_value=n / dt1, literal_vs_int=parity,
                    sample="%d passes over all %d images, literal fp32 restatement of QLinearConvOp (dequantize, im2col + "
                           "sequential-k GEMM, quantize), %d threads: %.1f s; one pass single-threaded: %.1f s" % (
                               reps, n, cores, dt, dt1))
    return res, roofline, cpu, plan.close


def bench_fusion(args, torch, pkg, qdq=False):
    import numpy as np
    ops = pkg.ops
    f32 = torch.float32
    torch.manual_seed(1)
    x = torch.randn(64, 1024, 1024, device="cuda")
    y = torch.empty_like(x)
    if qdq:
        prog = ops.fusion_program([("x", f32)], [("q", "QuantizeLinear", "x", 0.05, 0, "int8"),
                                                  ("y", "DequantizeLinear", "q", 0.05, 0)], [("y", f32)])
        ins, nbytes, name = [x], 2 * x.numel() * 4, "quantize_dequantize_fused"
    else:
        c = torch.randn_like(x)
        a = torch.randn(1024, device="cuda")
        b = torch.randn(1024, device="cuda")
        prog = ops.fusion_program(
            [("x", f32), ("a", f32), ("b", f32), ("c", f32)],
            [("t0", "Mul", "x", "a"), ("t1", "Add", "t0", "b"), ("t2", "Tanh", "t1"), ("t3", "Sigmoid", "c"),
             ("t4", "Mul", "t2", "t3"), ("t5", "Add", "t4", "x"), ("y", "Relu", "t5")], [("y", f32)])
        ins, nbytes, name = [x, a, b, c], 3 * x.numel() * 4 + 2 * 1024 * 4, "relu(tanh(x*a+b)*sigmoid(c)+x)"

    def step(timer):
        fn = lambda: ops.ElementWiseNvrtc(ins, 1, prog, 3, outs=[y])
        timer.wrap("ew", fn) if timer else fn()

    timer = KernelTimer(torch)
    sec = timed_steps(torch, step, args.steps, args.warmup, timer)
    cnt, ms = timer.totals()["ew"]
    achieved = nbytes / (ms / cnt * 1e-3) / 1e9
    roofline = dict(bound="hbm", kernel="fusion3_vec", achieved=achieved, peak=HBM_PEAK_GBS, unit="GB/s",
                    frac=achieved / HBM_PEAK_GBS, traffic=None, bytes_per_launch=nbytes, launch_us=ms / cnt * 1e3)
    res = dict(metric="GB/s FusionGroup %s fp32 [64,1024,1024] @1 GPU" % name, value=nbytes / sec / 1e9, unit="GB/s",
               ms_per_step=sec * 1e3, dtype="f32", config=dict(workload="fusion_" + ("qdq" if qdq else "chain"), elements=x.numel()))

    def cpu():
        from oracle import oracle as orc
        cores = orc.max_threads()
        orc.set_threads(cores)
        rows = 16 * 1024
        xs = x.view(-1, 1024)[:rows].cpu().numpy()
        t0 = time.perf_counter()
        if qdq:
            orc.dequantize_linear(orc.quantize_linear_multipass(xs, 0.05, 0, np.int8), 0.05, 0, multipass=True)
        else:
            cs = ins[3].view(-1, 1024)[:rows].cpu().numpy()
            orc.run_chain([("t0", "Mul", "x", "a"), ("t1", "Add", "t0", "b"), ("t2", "Tanh", "t1"),
                           ("t3", "Sigmoid", "c"), ("t4", "Mul", "t2", "t3"), ("t5", "Add", "t4", "x"),
                           ("y", "Relu", "t5")], dict(x=xs, a=ins[1].cpu().numpy(), b=ins[2].cpu().numpy(), c=cs))
        dt = time.perf_counter() - t0
        orc.set_threads(1)
        frac = rows * 1024 / x.numel()
        return dict(value=nbytes * frac / dt / 1e9, unit="GB/s", cores=cores, kind="port",
                    sample="%d of %d rows, op-by-op fp32 passes with temporaries, %d threads, %.2f s" % (
                        rows, x.numel() // 1024, cores, dt))
    return res, roofline, cpu, (lambda: None)


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one MI355X; this path has no multi-GPU leg (inference is data parallel over the "
              "batch and every GPU box here has one GPU).  Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    import torch
    import __graft_entry__ as entry
    pkg = entry.load_package()
    pkg.capi.init(0)
    if args.workload in ("resnet50", "mobilenetv2"):
        res, roofline, cpu, close = bench_resnet50(args, torch, pkg, mobilenet=args.workload == "mobilenetv2")
    elif args.workload == "conv3x3":
        res, roofline, cpu, close = bench_conv3x3(args, torch, pkg)
    else:
        res, roofline, cpu, close = bench_fusion(args, torch, pkg, qdq=args.workload == "qdq")
    if args.copy_probe_mib:
        n = args.copy_probe_mib * (1 << 20) // 4
        src = torch.ones(n, dtype=torch.float32, device="cuda")
        code = pkg.ops.fusion_program([("x", torch.float32)], [("y", "Identity", "x")], [("y", torch.float32)])
        pkg.ops.ElementWiseNvrtc([src], 1, code, 9999)
        torch.cuda.synchronize()
    others = None
    if args.workload == "resnet50" and not args.no_other_workloads and not args.batch and not args.no_graph:
        # the other configurations, shortly, so that one run reports all of them (their own --workload runs time them longer)
        import copy
        close()
        close = lambda: None
        others = []
        for name in ("conv3x3", "fusion", "qdq", "mobilenetv2"):
            a2 = copy.copy(args)
            a2.workload, a2.steps, a2.warmup = name, 10, 3
            torch.cuda.empty_cache()
            if name == "mobilenetv2":
                r2, roof2, _cpu2, close2 = bench_resnet50(a2, torch, pkg, mobilenet=True)
            elif name == "conv3x3":
                r2, roof2, _cpu2, close2 = bench_conv3x3(a2, torch, pkg)
            else:
                r2, roof2, _cpu2, close2 = bench_fusion(a2, torch, pkg, qdq=name == "qdq")
            close2()
            others.append(dict(workload=r2["config"]["workload"], metric=r2["metric"], value=r2["value"], unit=r2["unit"],
                               ms_per_step=r2["ms_per_step"], steps=a2.steps, warmup=a2.warmup,
                               roofline=dict(bound=roof2["bound"], kernel=roof2["kernel"], frac=roof2["frac"], achieved=roof2["achieved"],
                                             unit=roof2["unit"], kernel_us=roof2.get("launch_us", roof2.get("kernel_ms_per_step", 0.0) * 1e3 if "kernel_ms_per_step" in roof2 else None))))
    out = dict(res)
    if others is not None:
        out["other_workloads"] = others
    out.update(n_gpus=1, steps=args.steps, warmup=args.warmup, higher_is_better=True, scaling="weak", vs_baseline=None,
               data="synthetic", roofline=roofline)
    if not args.no_cpu_baseline:
        model, ncpu = cpu_info()
        cb = cpu()
        cb["host"] = "%s, %d logical CPUs visible" % (model, ncpu)
        out["cpu_baseline"] = cb
    close()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
