"""Quantized networks as hand-built ChxVM-style programs: the ResNet-50 int8 QDQ
configuration the headline metric is quoted on and the MobileNetV2 configuration with its
depthwise convolutions, in the op vocabulary of this path.

A program is a list of instructions over named values; every instruction is one op
of the path (QuantizeLinear, QLinearConv, MaxPool, FusionGroup Add+Relu, AveragePool,
DequantizeLinear).  `build_resnet50` only constructs data (weights, scales, the
instruction list); executing it is the job of `DeviceRunner` (MI355X, through the C
ABI) or of a reference executor supplied by the tests and the benchmark.

Construction follows the reference where it defines the step:
  architecture            scripts/resnet50.py:10-107 (stride on the first 1x1 of a
                          down-sampling bottleneck, 7x7/2 stem with bias, 3x3/2
                          max-pool with cover_all, 7x7 average pool, FC 2048->1000)
  BatchNorm folding       compiler/merge.cc:142-211: s = gamma / sqrt(var + eps),
                          w' = w * s, b' = (b - mean) * s + beta
  weight quantization     compiler/quantize.cc:77-81, per output channel:
                          scale = 2 max|w| / 254, q = rint(w / scale), zero point 0
  activation quantization compiler/quantize.cc:84-86 on the min/max of one seeded
                          batch: scale = (max - min) / 255 with min <= 0 <= max,
                          zero_point = rint(-min / scale), uint8
Bias is int32 at scale x_scale * w_scale[oc] (the ONNX QLinearConv definition).
A Relu after a convolution is folded into the convolution's output quantization:
the calibrated post-Relu range starts at 0, so the zero point is 0 and the uint8
saturation of QLinearConv is the Relu (Q(Relu(DQ(q))) == q for every code).
"""
import numpy as np
import torch
import torch.nn.functional as F

EPS = 2e-5  # chainer.links.BatchNormalization default


def _he_normal(rng, shape):
    fan_in = int(np.prod(shape[1:]))
    return (rng.standard_normal(shape) * np.sqrt(2.0 / fan_in)).astype(np.float32)


def _fold_bn(rng, w, b):
    oc = w.shape[0]
    gamma = rng.uniform(0.5, 1.5, oc).astype(np.float32)
    beta = (rng.standard_normal(oc) * 0.1).astype(np.float32)
    mean = (rng.standard_normal(oc) * 0.1).astype(np.float32)
    var = rng.uniform(0.5, 1.5, oc).astype(np.float32)
    s = (gamma / np.sqrt(var + np.float32(EPS))).astype(np.float32)
    w2 = (w * s[:, None, None, None]).astype(np.float32)
    b0 = np.zeros(oc, np.float32) if b is None else b
    b2 = ((b0 - mean) * s + beta).astype(np.float32)
    return w2, b2


def quantize_weights_per_channel(w):
    """compiler/quantize.cc:77-81 applied per output channel (QuantizeWeightConvolution)."""
    oc = w.shape[0]
    flat = w.reshape(oc, -1)
    rmin = np.minimum(flat.min(axis=1), 0).astype(np.float32)
    rmax = np.maximum(flat.max(axis=1), 0).astype(np.float32)
    max_range = np.maximum(np.abs(rmin), np.abs(rmax)).astype(np.float32)
    scale = (max_range * np.float32(2) / np.float32(254)).astype(np.float32)
    scale = np.where(scale == 0, np.float32(1), scale).astype(np.float32)
    q = np.rint(w / scale[:, None, None, None]).astype(np.int8)
    return q, scale


def activation_qparams(t):
    """compiler/quantize.cc:84-86: uint8, range widened to contain 0."""
    rmin = min(float(t.min()), 0.0)
    rmax = max(float(t.max()), 0.0)
    scale = np.float32((np.float32(rmax) - np.float32(rmin)) / np.float32(255)) if rmin != rmax else np.float32(1)
    zp = int(np.rint((0 - np.float32(rmin)) / scale))
    return scale, zp


class ConvLayer(object):
    def __init__(self, name, w, b, stride, pad, group=1):
        self.name, self.wf, self.bf, self.stride, self.pad, self.group = name, w, b, stride, pad, group
        self.wq, self.w_scale = quantize_weights_per_channel(w)
        self.w_zp = np.zeros(w.shape[0], np.int8)
        self.x_scale = self.x_zp = self.y_scale = self.y_zp = None
        self.bias_q = None

    def finish(self):
        s = (np.float32(self.x_scale) * self.w_scale).astype(np.float32)
        self.bias_q = np.rint(self.bf / s).astype(np.int64).clip(-2 ** 31, 2 ** 31 - 1).astype(np.int32)

    def macs(self, out_shape):
        n, oc, oh, ow = out_shape
        return n * oh * ow * oc * int(np.prod(self.wf.shape[1:]))


def build_resnet50(batch=64, image=224, seed=3, width=64, blocks=(3, 4, 6, 3), classes=1000, device=None):
    """Returns a dict: program (instruction list), convs (name -> ConvLayer), qparams
    (value name -> (scale, zero_point)), input (the seeded fp32 batch), shapes, macs.

    `width`, `blocks`, `image`, `classes` shrink the network for tests; the defaults are
    ResNet-50 v1."""
    rng = np.random.default_rng(seed)
    dev = device or ("cuda" if torch.cuda.is_available() else "cpu")
    x = rng.standard_normal((batch, 3, image, image)).astype(np.float32)
    program, convs, qparams, shapes = [], {}, {}, {}
    fvals = {"x": torch.from_numpy(x).to(dev)}

    def note(name):
        qparams[name] = activation_qparams(fvals[name])
        shapes[name] = tuple(fvals[name].shape)

    def conv(name, src, dst, cin, cout, k, stride, pad, relu, bias=False):
        w = _he_normal(rng, (cout, cin, k, k))
        b = (rng.standard_normal(cout) * 0.1).astype(np.float32) if bias else None
        w, b = _fold_bn(rng, w, b)
        layer = ConvLayer(name, w, b, stride, pad)
        convs[name] = layer
        # calibration runs the float network with the weights the quantized one represents
        wd = torch.from_numpy(layer.wq.astype(np.float32) * layer.w_scale[:, None, None, None]).to(dev)
        y = F.conv2d(fvals[src], wd, torch.from_numpy(b).to(dev), stride=stride, padding=pad)
        fvals[dst] = F.relu(y) if relu else y
        note(dst)
        layer.x_scale, layer.x_zp = qparams[src]
        layer.y_scale, layer.y_zp = qparams[dst]
        layer.finish()
        program.append(("QLinearConv", dst, src, name))

    note("x")
    program.append(("QuantizeLinear", "x_q", "x") + qparams["x"])
    fvals["x_q"] = fvals["x"]
    qparams["x_q"], shapes["x_q"] = qparams["x"], shapes["x"]
    conv("conv1", "x_q", "stem", 3, width, 7, 2, 3, relu=True, bias=True)
    fvals["pool1"] = F.max_pool2d(fvals["stem"], 3, 2, 0, ceil_mode=True)
    qparams["pool1"], shapes["pool1"] = qparams["stem"], tuple(fvals["pool1"].shape)
    program.append(("MaxPool", "pool1", "stem", 3, 2, 0, True))

    cur, cin = "pool1", width
    for si, nblk in enumerate(blocks):
        ch = width * (2 ** si)
        cout = ch * 4
        for bi in range(nblk):
            p = "res%d_%d" % (si + 2, bi)
            stride = 2 if (bi == 0 and si > 0) else 1
            conv(p + "_c1", cur, p + "_a", cin, ch, 1, stride, 0, relu=True)
            conv(p + "_c2", p + "_a", p + "_b", ch, ch, 3, 1, 1, relu=True)
            conv(p + "_c3", p + "_b", p + "_c", ch, cout, 1, 1, 0, relu=False)
            if bi == 0:
                conv(p + "_c4", cur, p + "_s", cin, cout, 1, stride, 0, relu=False)
                short = p + "_s"
            else:
                short = cur
            fvals[p] = F.relu(fvals[p + "_c"] + fvals[short])
            note(p)
            program.append(("AddRelu", p, p + "_c", short))
            for tmp in (p + "_a", p + "_b", p + "_c", p + "_s", cur):
                fvals.pop(tmp, None)   # calibration activations no longer needed
            cur, cin = p, cout
    k = fvals[cur].shape[2]
    fvals["gap"] = F.avg_pool2d(fvals[cur], k, 1)
    note("gap")
    program.append(("AveragePool", "gap", cur, int(k)))
    conv("fc", "gap", "logits_q", cin, classes, 1, 1, 0, relu=False, bias=True)
    program.append(("DequantizeLinear", "logits", "logits_q") + qparams["logits_q"])
    shapes["logits"] = shapes["logits_q"]
    total_macs = 0
    for ins in program:
        if ins[0] == "QLinearConv":
            total_macs += convs[ins[3]].macs(shapes[ins[1]])
    return dict(program=program, convs=convs, qparams=qparams, shapes=shapes, input=x, macs=total_macs,
                float_logits=fvals["logits_q"].detach().cpu().numpy())


# MobileNetV2-1.0 (Sandler et al. 2018, table 2): expansion t, output channels c, repeats n, stride s
MOBILENETV2_BLOCKS = ((1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 3, 2), (6, 64, 4, 2), (6, 96, 3, 1), (6, 160, 3, 2),
                      (6, 320, 1, 1))


def build_mobilenetv2(batch=128, image=224, seed=4, blocks=MOBILENETV2_BLOCKS, stem=32, head=1280, classes=1000,
                      device=None):
    """MobileNetV2 as a QDQ program: 3x3/2 stem, inverted residual blocks (1x1 expansion,
    depthwise 3x3, linear 1x1 projection, residual Add where shapes agree), 1x1 head, global
    average pool, classifier.  Kaiming-normal weights with BatchNorm folded; every ReLU6 is
    folded into the output quantization of its convolution (the calibrated range of a
    post-ReLU6 tensor is [0, <=6], zero point 0, so uint8 saturation is the clipping); the
    linear projections and the residual sums get asymmetric uint8 ranges.  `blocks`, `stem`,
    `head`, `image`, `classes` shrink the network for tests."""
    rng = np.random.default_rng(seed)
    dev = device or ("cuda" if torch.cuda.is_available() else "cpu")
    x = rng.standard_normal((batch, 3, image, image)).astype(np.float32)
    program, convs, qparams, shapes = [], {}, {}, {}
    fvals = {"x": torch.from_numpy(x).to(dev)}

    def note(name):
        qparams[name] = activation_qparams(fvals[name])
        shapes[name] = tuple(fvals[name].shape)

    def conv(name, src, dst, cin, cout, k, stride, pad, relu6, group=1, bias=False):
        w = _he_normal(rng, (cout, cin // group, k, k))
        b = (rng.standard_normal(cout) * 0.1).astype(np.float32) if bias else None
        w, b = _fold_bn(rng, w, b)
        layer = ConvLayer(name, w, b, stride, pad, group)
        convs[name] = layer
        wd = torch.from_numpy(layer.wq.astype(np.float32) * layer.w_scale[:, None, None, None]).to(dev)
        y = F.conv2d(fvals[src], wd, torch.from_numpy(b).to(dev), stride=stride, padding=pad, groups=group)
        fvals[dst] = F.relu6(y) if relu6 else y
        note(dst)
        layer.x_scale, layer.x_zp = qparams[src]
        layer.y_scale, layer.y_zp = qparams[dst]
        layer.finish()
        program.append(("QLinearConv", dst, src, name))

    note("x")
    program.append(("QuantizeLinear", "x_q", "x") + qparams["x"])
    fvals["x_q"] = fvals["x"]
    qparams["x_q"], shapes["x_q"] = qparams["x"], shapes["x"]
    conv("stem", "x_q", "f0", 3, stem, 3, 2, 1, relu6=True)
    cur, cin, bi = "f0", stem, 0
    for t, c, n, s_ in blocks:
        for i in range(n):
            bi += 1
            p = "b%d" % bi
            stride = s_ if i == 0 else 1
            hidden = cin * t
            src = cur
            if t != 1:
                conv(p + "_expand", src, p + "_e", cin, hidden, 1, 1, 0, relu6=True)
                src = p + "_e"
            conv(p + "_dw", src, p + "_d", hidden, hidden, 3, stride, 1, relu6=True, group=hidden)
            conv(p + "_project", p + "_d", p + "_p", hidden, c, 1, 1, 0, relu6=False)
            out = p + "_p"
            if stride == 1 and cin == c:
                fvals[p] = fvals[p + "_p"] + fvals[cur]
                note(p)
                program.append(("Add", p, p + "_p", cur))
                out = p
            for tmp in (p + "_e", p + "_d", cur) + ((p + "_p",) if out != p + "_p" else ()):
                fvals.pop(tmp, None)
            cur, cin = out, c
    conv("head", cur, "head", cin, head, 1, 1, 0, relu6=True)
    k = fvals["head"].shape[2]
    fvals["gap"] = F.avg_pool2d(fvals["head"], k, 1)
    note("gap")
    program.append(("AveragePool", "gap", "head", int(k)))
    conv("fc", "gap", "logits_q", head, classes, 1, 1, 0, relu6=False, bias=True)
    program.append(("DequantizeLinear", "logits", "logits_q") + qparams["logits_q"])
    shapes["logits"] = shapes["logits_q"]
    total_macs = 0
    dw_bytes = 0
    for ins in program:
        if ins[0] == "QLinearConv":
            layer = convs[ins[3]]
            total_macs += layer.macs(shapes[ins[1]])
            if layer.group > 1:
                # algorithmic bytes of a depthwise layer: activations in and out once, nine weights per channel
                dw_bytes += int(np.prod(shapes[ins[2]])) + int(np.prod(shapes[ins[1]])) + 9 * layer.group
    return dict(program=program, convs=convs, qparams=qparams, shapes=shapes, input=x, macs=total_macs,
                depthwise_bytes=dw_bytes, float_logits=fvals["logits_q"].detach().cpu().numpy())


def add_program(ops, qa, qb, qy):
    """FusionGroup text for Q(DQ(a) + DQ(b)) on uint8 tensors (a residual sum without Relu)."""
    u8 = torch.uint8
    return ops.fusion_program(
        [("a", u8), ("b", u8)],
        [("fa", "DequantizeLinear", "a", "0x%08x" % np.float32(qa[0]).view(np.uint32), qa[1]),
         ("fb", "DequantizeLinear", "b", "0x%08x" % np.float32(qb[0]).view(np.uint32), qb[1]),
         ("s", "Add", "fa", "fb"),
         ("q", "QuantizeLinear", "s", "0x%08x" % np.float32(qy[0]).view(np.uint32), qy[1], "uint8")],
        [("q", u8)])


def add_relu_program(ops, qa, qb, qy):
    """FusionGroup text for Q(Relu(DQ(a) + DQ(b))) on uint8 tensors."""
    u8 = torch.uint8
    return ops.fusion_program(
        [("a", u8), ("b", u8)],
        [("fa", "DequantizeLinear", "a", "0x%08x" % np.float32(qa[0]).view(np.uint32), qa[1]),
         ("fb", "DequantizeLinear", "b", "0x%08x" % np.float32(qb[0]).view(np.uint32), qb[1]),
         ("s", "Add", "fa", "fb"), ("r", "Relu", "s"),
         ("q", "QuantizeLinear", "r", "0x%08x" % np.float32(qy[0]).view(np.uint32), qy[1], "uint8")],
        [("q", u8)])


def pair_convolutions(program, convs):
    """The program with every two QLinearConv that read the same value with the same geometry (the main-path and the
    shortcut convolution of a down-sampling block) replaced by one instruction
    ("QLinearConvPair", out1, x, conv1, out2, conv2) at the place of the first: one launch computes both
    (chx_hip_qconv_plan_run_pair).  The first one's output channels must be a multiple of 64."""
    out, taken = [], set()
    for i, ins in enumerate(program):
        if i in taken:
            continue
        if ins[0] == "QLinearConv":
            a = convs[ins[3]]
            for j in range(i + 1, len(program)):
                other = program[j]
                if other[0] != "QLinearConv" or other[2] != ins[2] or j in taken:
                    continue
                b = convs[other[3]]
                same = (a.stride, a.pad, a.group, a.wq.shape[1:]) == (b.stride, b.pad, 1, b.wq.shape[1:])
                if same and a.wq.shape[0] % 64 == 0 and a.wq.shape[1] >= 16:
                    out.append(("QLinearConvPair", ins[1], ins[2], ins[3], other[1], other[3]))
                    taken.add(j)
                    break
            else:
                out.append(ins)
            continue
        out.append(ins)
    return out


def minus_128_values(program, convs, fused_into):
    """The values of `program` that can be stored as code - 128 in int8 arrays (CHX_HIP_STORE_MINUS_128): written by the
    matrix-core convolution kernel (a QLinearConv that is not grouped and has at least 16 input channels, a pair of them,
    or the residual sum inside one) or by the depthwise 3x3 kernel, and read only by convolutions that are not grouped (the
    depthwise kernel gains nothing from the storage), as their input or as the residual operand of a sum that one of
    them computes.  A reading convolution whose window leaves the image by more than one row or column
    must find the padding value, its input's zero point, stored as the byte 0 (a uint8 zero point of 128), or it does
    not run with the padding that costs nothing; a value with such a reader and another zero point keeps its uint8 array.
    `fused_into`: convolution result -> the Add instruction computed inside that convolution."""
    fused_adds = set(add[1] for add in fused_into.values())
    producers = {}
    for ins in program:
        c = convs[ins[3]] if ins[0] == "QLinearConv" else None
        depthwise = c is not None and c.group > 1 and c.group % 16 == 0 and tuple(c.wq.shape) == (c.group, 1, 3, 3)
        if c is not None and ((c.group == 1 and c.wq.shape[1] >= 16) or depthwise):
            producers[fused_into[ins[1]][1] if ins[1] in fused_into else ins[1]] = ins
        if ins[0] == "QLinearConvPair":
            producers[ins[1]] = producers[ins[4]] = ins
    keep = set()
    for name in producers:
        ok, readers = True, 0
        for ins in program:
            if ins[0] in ("QLinearConv", "QLinearConvPair"):
                if ins[2] == name:
                    readers += 1
                    c = convs[ins[3]]
                    if (c.pad > 1 and c.x_zp != 128) or c.group != 1:
                        ok = False
            elif ins[0] in ("Add", "AddRelu") and ins[1] in fused_adds:
                # computed inside a convolution: `name` may be its residual operand, not the convolution's own result
                conv_out = [k for k, add in fused_into.items() if add[1] == ins[1]][0]
                if name in ins[2:4] and name != conv_out:
                    readers += 1
            elif name in [a for a in ins[2:4] if isinstance(a, str)]:
                ok = False
        if ok and readers:
            keep.add(name)
    return keep


class DeviceRunner(object):
    """Runs a program on the MI355X: weights resident, one plan per QLinearConv, every
    activation channels-last, all intermediate buffers allocated once."""

    def __init__(self, model, pkg, fuse_residual=False, reuse_buffers=False, pair_convs=False, minus_128=False):
        """fuse_residual: a QLinearConv whose only reader is the residual Add(+Relu) of its block runs
        as one kernel with it; the convolution's own output is then not materialised.
        reuse_buffers: a value's memory goes back to a pool after its last reader and is handed to later
        values (as the VM's allocator does when the program frees a slot): the working set of a step is
        then a few tensors instead of every tensor of the network, and run() returns only values that are
        still live at the end (the program's last result is).
        pair_convs: two convolutions of the same value with the same geometry run as one launch (pair_convolutions);
        minus_128: values that only convolutions read are stored as code - 128 in int8 arrays (minus_128_values; the
        entries of run()'s result for them are int8 tensors), which spares the reading kernel the sign flips;
        self.program is the instruction list the runner executes."""
        self.m, self.ops, self.capi = model, pkg.ops, pkg.capi
        self.fused_into = {}   # conv output name -> the Add instruction that absorbs it
        program = pair_convolutions(model["program"], model["convs"]) if pair_convs else model["program"]
        self.program = program
        if fuse_residual:
            for i, ins in enumerate(program):
                if ins[0] in ("AddRelu", "Add") and i > 0:
                    prev = program[i - 1]
                    readers = sum(1 for other in program if prev[1] in other[2:4] and other[0] != "QuantizeLinear")
                    if prev[0] == "QLinearConv" and prev[1] in ins[2:4] and readers == 1 and model["convs"][prev[3]].group == 1:
                        self.fused_into[prev[1]] = ins
        self.minus_128 = minus_128_values(program, model["convs"], self.fused_into) if minus_128 else set()
        self.dev = {}
        self.plans = {}
        self.bufs = {}
        self.fusion = {}
        self.full = {}
        self.reuse_buffers = reuse_buffers
        for name, c in model["convs"].items():
            t = [torch.from_numpy(a).cuda() for a in (c.wq, c.w_scale, c.w_zp, c.bias_q)]
            self.dev[name] = t
            self.plans[name] = self.ops.QLinearConvPlan(t[0], t[1], t[2], t[3], strides=(c.stride, c.stride),
                                                        pads=(c.pad, c.pad), group=c.group)
        for ins in program:
            if ins[0] == "QLinearConvPair":
                # both filter sets one after the other along the output channels
                t = [torch.cat([a, b]) for a, b in zip(self.dev[ins[3]], self.dev[ins[5]])]
                c = model["convs"][ins[3]]
                self.dev[ins[3] + "+" + ins[5]] = t
                self.plans[ins[3] + "+" + ins[5]] = self.ops.QLinearConvPlan(t[0], t[1], t[2], t[3], strides=(c.stride, c.stride),
                                                                          pads=(c.pad, c.pad), group=1)
        # raw byte blocks: fresh per value, or from the pool of released ones (the smallest that fits)
        free_blocks = []

        def take(nbytes):
            fits = [i for i, b in enumerate(free_blocks) if b.numel() >= nbytes]
            if reuse_buffers and fits:
                best = free_blocks.pop(min(fits, key=lambda i: free_blocks[i].numel()))
                best[:nbytes].zero_()
                return best
            return torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
        last_use = {}
        for i, ins in enumerate(program):
            for name in ins[2:4]:
                if isinstance(name, str):
                    last_use[name] = i
        block_of = {}

        def make(out, kind):
            shp = model["shapes"][out]
            if kind == "DequantizeLinear":
                n = int(np.prod(shp)) * 4
                block_of[out] = take(n)
                self.bufs[out] = block_of[out][:n].view(torch.float32).view(shp)
            elif kind == "QuantizeLinear":
                # the network input stays NCHW like the fp32 tensor it is quantized from (one flat,
                # fully coalesced pass); the 3-channel stem reads it through its im2col step
                n = int(np.prod(shp))
                block_of[out] = take(n)
                self.bufs[out] = block_of[out][:n].view(shp)
            else:
                # channels-last with the pixel pitch rounded up to 16 bytes, so that every pixel is a
                # whole number of aligned 16-byte vectors also for channel counts like 24
                n, c, h, w = shp
                pitch = (c + 15) // 16 * 16
                block_of[out] = take(n * h * w * pitch)
                full = block_of[out][:n * h * w * pitch].view(n, h, w, pitch)
                if out in self.minus_128:
                    full = full.view(torch.int8)
                self.bufs[out] = full[..., :c].permute(0, 3, 1, 2)
                # element-wise groups run over the padded pixels as they lie in memory (dense)
                self.full[out] = full.permute(0, 3, 1, 2)
        for i, ins in enumerate(program):
            kind, out = ins[0], ins[1]
            if kind == "QLinearConv" and out in self.fused_into:
                add = self.fused_into[out]
                make(add[1], add[0])     # the fused convolution writes the sum here, one instruction early
            elif out not in self.bufs:
                make(out, kind)
            if kind == "QLinearConvPair":
                make(ins[4], kind)
            q = model["qparams"]
            if kind == "AddRelu":
                self.fusion[out] = add_relu_program(self.ops, q[ins[2]], q[ins[3]], q[out])
            if kind == "Add":
                self.fusion[out] = add_program(self.ops, q[ins[2]], q[ins[3]], q[out])
            if reuse_buffers:
                for name in set(n for n in ins[2:4] if isinstance(n, str)):
                    if last_use.get(name) == i and name in block_of:
                        free_blocks.append(block_of.pop(name))
        self.live_at_end = set(block_of)

    def launch(self, fid, v):
        """Launches instruction number `fid` of the program on the values `v` (name -> tensor)."""
        ops, q, m = self.ops, self.m["qparams"], self.m
        ins = self.program[fid]
        kind, out = ins[0], ins[1]
        buf = self.bufs.get(out)   # none for a convolution whose result only exists inside the fused residual sum
        S = self.minus_128
        zp_of = lambda name, zp: zp - 128 if name in S else zp                    # an int8 array of codes minus 128
        dt_of = lambda name: torch.int8 if name in S else torch.uint8
        fl_of = lambda name: self.capi.BIAS_ONNX_INT32 | (self.capi.STORE_MINUS_128 if name in S else 0)
        if kind == "QuantizeLinear":
            ops.QuantizeLinear(v[ins[2]], ins[3], ins[4], torch.uint8, out=buf)
        elif kind == "QLinearConv" and out in self.fused_into:
            add = self.fused_into[out]
            other = add[3] if add[2] == out else add[2]
            c = m["convs"][ins[3]]
            # DequantizeLinear(a) + DequantizeLinear(b) is commutative bit for bit, so the
            # convolution may be either operand of the Add
            self.plans[ins[3]].run_add(v[ins[2]], c.x_scale, zp_of(ins[2], c.x_zp), c.y_scale, c.y_zp, v[other], q[other][0],
                                       zp_of(other, q[other][1]), q[add[1]][0], q[add[1]][1], add[0] == "AddRelu", torch.uint8,
                                       flags=fl_of(add[1]), out=self.bufs[add[1]])
            return None
        elif kind in ("AddRelu", "Add") and (ins[2] in self.fused_into or ins[3] in self.fused_into):
            pass   # written by the fused convolution
        elif kind == "QLinearConv":
            c = m["convs"][ins[3]]
            self.plans[ins[3]].run(v[ins[2]], c.x_scale, zp_of(ins[2], c.x_zp), c.y_scale, c.y_zp, dt_of(out), flags=fl_of(out), out=buf)
        elif kind == "QLinearConvPair":
            c1, c2 = m["convs"][ins[3]], m["convs"][ins[5]]
            self.plans[ins[3] + "+" + ins[5]].run_pair(
                v[ins[2]], c1.x_scale, zp_of(ins[2], c1.x_zp), c1.wq.shape[0], c1.y_scale, c1.y_zp, c2.y_scale, c2.y_zp,
                flags=(fl_of(out), fl_of(ins[4])), outs=(buf, self.bufs[ins[4]]))
            v[ins[4]] = self.bufs[ins[4]]
        elif kind == "MaxPool":
            ops.MaxPoolQ8(v[ins[2]], (ins[3], ins[3]), (ins[4], ins[4]), (ins[5], ins[5]), ins[6], out=buf)
        elif kind in ("AddRelu", "Add"):
            ops.ElementWiseNvrtc([self.full[ins[2]], self.full[ins[3]]], 1, self.fusion[out], fid, outs=[self.full[out]])
        elif kind == "AveragePool":
            ops.AveragePoolQ8(v[ins[2]], q[ins[2]][0], q[ins[2]][1], (ins[3], ins[3]), (1, 1), (0, 0), q[out][0],
                              q[out][1], out=buf)
        elif kind == "DequantizeLinear":
            ops.DequantizeLinear(v[ins[2]], ins[3], ins[4], out=buf)
        else:
            raise ValueError(kind)
        return buf

    def run(self, x):
        v = {"x": x}
        for fid, ins in enumerate(self.program):
            buf = self.launch(fid, v)
            if buf is not None:
                v[ins[1]] = buf
        if self.reuse_buffers:
            return {k: t for k, t in v.items() if k == "x" or k in self.live_at_end}
        return v

    def capture(self, x):
        """Records one pass of the program into a HIP graph (after a warm-up pass that
        compiles the fused kernels and sizes every plan's scratch) and returns a callable that
        replays it: the launch-bound instruction sequence then costs one graph launch."""
        self.run(x)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            values = self.run(x)
        self._graph = graph

        def replay():
            graph.replay()
            return values
        return replay

    def close(self):
        self._graph = None
        for p in self.plans.values():
            p.close()


def program_to_chxvm(model, vm, ops, keep=("logits",)):
    """The op program as a serialized ChxVMProgramProto, in the form the reference's compiler gives
    a QDQ graph: QuantizeLinear / QLinearConv / DequantizeLinear instructions with constant
    operands, pools between a DequantizeLinear and a QuantizeLinear, residual sums as
    ElementWiseNvrtc FusionGroups.  `vm` is the chxvm module, `ops` the ops module.
    QLinearConv biases are int32 at scale x_scale * w_scale: run with the option
    qlinearconv_bias = onnx_int32.  `keep` names the values that become program outputs."""
    b = vm.ProgramBuilder()
    q = model["qparams"]
    slot = {}

    def scalars(name):
        return b.scalar(float(q[name][0]), "float32"), b.scalar(int(q[name][1]), "uint8")
    for fid, ins in enumerate(model["program"]):
        kind, out = ins[0], ins[1]
        if kind == "QuantizeLinear":
            slot[ins[2]] = b.input(ins[2], "float32", model["shapes"][ins[2]])
            s, z = b.scalar(float(ins[3]), "float32"), b.scalar(int(ins[4]), "uint8")
            slot[out] = b.QuantizeLinear(slot[ins[2]], s, z, debug_info=out)
        elif kind == "QLinearConv":
            c = model["convs"][ins[3]]
            xs, xz = b.scalar(float(c.x_scale), "float32"), b.scalar(int(c.x_zp), "uint8")
            ys, yz = b.scalar(float(c.y_scale), "float32"), b.scalar(int(c.y_zp), "uint8")
            slot[out] = b.QLinearConv(slot[ins[2]], xs, xz, b.constant(c.wq), b.constant(c.w_scale), b.constant(c.w_zp), ys, yz,
                                      b.constant(c.bias_q), [c.stride, c.stride], [c.pad, c.pad], c.group, "", debug_info=out)
        elif kind in ("MaxPool", "AveragePool"):
            s_in, z_in = scalars(ins[2])
            f = b.DequantizeLinear(slot[ins[2]], s_in, z_in, debug_info=out)
            g = b.new_slot()
            if kind == "MaxPool":
                k, st, pad, cover_all = ins[3], ins[4], ins[5], ins[6]
                b.add_raw("MaxPool", [("ARRAY", f), ("INTS", [k, k]), ("INTS", [st, st]), ("INTS", [pad, pad]),
                                      ("INT", 1 if cover_all else 0), ("STRING", "NOTSET")], [g, -1], debug_info=out)
            else:
                k = ins[3]
                b.add_raw("AveragePool", [("ARRAY", f), ("INTS", [k, k]), ("INTS", [1, 1]), ("INTS", [0, 0]), ("INT", 0)],
                          [g, -1], debug_info=out)
            s_out, z_out = scalars(out)
            slot[out] = b.QuantizeLinear(g, s_out, z_out, debug_info=out)
            b.Free(f)
            b.Free(g)
        elif kind in ("AddRelu", "Add"):
            make = add_relu_program if kind == "AddRelu" else add_program
            code = make(ops, q[ins[2]], q[ins[3]], q[out])
            slot[out] = b.ElementWiseNvrtc([slot[ins[2]], slot[ins[3]]], 1, code, fid, num_list_outputs=1, debug_info=out)[0]
        elif kind == "DequantizeLinear":
            s, z = b.scalar(float(ins[3]), "float32"), b.scalar(int(ins[4]), "uint8")
            slot[out] = b.DequantizeLinear(slot[ins[2]], s, z, debug_info=out)
        else:
            raise ValueError(kind)
        # the compiler frees a value after its last reader (compiler/scheduler.cc, compiler/chxvm/emitter.cc)
        for name in ins[2:4]:
            if isinstance(name, str) and name in slot and name not in keep and not _still_needed(model["program"], ins, name):
                b.Free(slot[name])
    for name in keep:
        b.output(name, slot[name])
    return b


def program_to_onnx(model, onnx_lite, keep=("logits",)):
    """The op program as an ONNX QDQ graph (serialized ModelProto): QuantizeLinear / QLinearConv /
    DequantizeLinear nodes with initializers, pools between a DequantizeLinear and a QuantizeLinear,
    residual sums as DequantizeLinear, DequantizeLinear, Add, [Relu], QuantizeLinear -- what a
    quantization tool leaves and the compiler side here takes (fusion pass, emitter)."""
    g = onnx_lite.Graph()
    g.name = "network"
    q = model["qparams"]
    inits = {}

    def const(name, value):
        inits[name] = np.asarray(value)
        return name

    def qp(name):
        return [const(name + "_scale", np.float32(q[name][0])), const(name + "_zp", np.uint8(q[name][1]))]
    nodes = []
    for ins in model["program"]:
        kind, out = ins[0], ins[1]
        if kind == "QuantizeLinear":
            g.inputs.append((ins[2], onnx_lite.FLOAT, list(model["shapes"][ins[2]])))
            nodes.append(onnx_lite.Node("QuantizeLinear", [ins[2], const(out + "_scale", np.float32(ins[3])), const(out + "_zp", np.uint8(ins[4]))],
                                        [out]))
        elif kind == "QLinearConv":
            c = model["convs"][ins[3]]
            n = ins[3]
            operands = [ins[2], const(n + "_xs", np.float32(c.x_scale)), const(n + "_xz", np.uint8(c.x_zp)), const(n + "_w", c.wq),
                        const(n + "_ws", c.w_scale), const(n + "_wz", c.w_zp), const(n + "_ys", np.float32(c.y_scale)),
                        const(n + "_yz", np.uint8(c.y_zp)), const(n + "_b", c.bias_q)]
            k = c.wq.shape[2]
            nodes.append(onnx_lite.Node("QLinearConv", operands, [out],
                                        {"strides": [c.stride, c.stride], "pads": [c.pad] * 4, "group": c.group, "kernel_shape": [k, k]}, name=n))
        elif kind in ("MaxPool", "AveragePool"):
            nodes.append(onnx_lite.Node("DequantizeLinear", [ins[2]] + qp(ins[2]), [out + "__f"]))
            if kind == "MaxPool":
                attrs = {"kernel_shape": [ins[3]] * 2, "strides": [ins[4]] * 2, "pads": [ins[5]] * 4, "chainer_cover_all": 1 if ins[6] else 0}
            else:
                attrs = {"kernel_shape": [ins[3]] * 2, "strides": [1, 1], "pads": [0] * 4}
            nodes.append(onnx_lite.Node(kind, [out + "__f"], [out + "__p"], attrs))
            nodes.append(onnx_lite.Node("QuantizeLinear", [out + "__p"] + qp(out), [out]))
        elif kind in ("AddRelu", "Add"):
            nodes.append(onnx_lite.Node("DequantizeLinear", [ins[2]] + qp(ins[2]), [out + "__fa"]))
            nodes.append(onnx_lite.Node("DequantizeLinear", [ins[3]] + qp(ins[3]), [out + "__fb"]))
            nodes.append(onnx_lite.Node("Add", [out + "__fa", out + "__fb"], [out + "__s"]))
            last = out + "__s"
            if kind == "AddRelu":
                nodes.append(onnx_lite.Node("Relu", [last], [out + "__r"]))
                last = out + "__r"
            nodes.append(onnx_lite.Node("QuantizeLinear", [last] + qp(out), [out]))
        elif kind == "DequantizeLinear":
            nodes.append(onnx_lite.Node("DequantizeLinear", [ins[2], const(out + "_scale", np.float32(ins[3])), const(out + "_zp", np.uint8(ins[4]))],
                                        [out]))
        else:
            raise ValueError(kind)
    g.nodes = nodes
    g.initializers = inits
    g.inputs += [(k, onnx_lite.ONNX_OF[v.dtype], list(v.shape)) for k, v in inits.items()]
    for name in keep:
        elem = onnx_lite.FLOAT if name == "logits" else onnx_lite.UINT8
        g.outputs.append((name, elem, list(model["shapes"][name])))
    return onnx_lite.make_model(g)


def slice_model(model, lo, hi):
    """The same program on images lo..hi-1 of the batch (weights and quantization parameters are
    shared; only the shapes and the input change)."""
    sub = dict(model)
    sub["shapes"] = {k: (hi - lo,) + tuple(v[1:]) for k, v in model["shapes"].items()}
    sub["input"] = model["input"][lo:hi]
    return sub


class ConcurrentRunner(object):
    """Runs the batch as `parts` independent slices, each on its own stream with its own plans and
    buffers.  Inference is independent per image, so the values are those of the whole-batch
    run; the point is occupancy: one ResNet layer at batch 64 is a few hundred work-groups, too
    few to keep 256 compute units busy through its ramp and tail, and the slices' kernels fill
    each other's gaps."""

    def __init__(self, model, pkg, parts=2, fuse_residual=False):
        n = model["shapes"]["x"][0]
        bounds = [n * i // parts for i in range(parts + 1)]
        self.slices = [(bounds[i], bounds[i + 1]) for i in range(parts) if bounds[i + 1] > bounds[i]]
        self.runners = [DeviceRunner(slice_model(model, lo, hi), pkg, fuse_residual) for lo, hi in self.slices]
        self.streams = [torch.cuda.Stream() for _ in self.runners]

    def run(self, x):
        cur = torch.cuda.current_stream()
        outs = []
        for (lo, hi), r, st in zip(self.slices, self.runners, self.streams):
            st.wait_stream(cur)
            with torch.cuda.stream(st):
                outs.append(r.run(x[lo:hi]))
        for st in self.streams:
            cur.wait_stream(st)
        return outs

    def capture(self, x):
        self.run(x)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            values = self.run(x)
        self._graph = graph

        def replay():
            graph.replay()
            return values
        return replay

    def close(self):
        self._graph = None
        for r in self.runners:
            r.close()


def conv_layer_table(model, fuse_residual=True, pair_convs=False):
    """One row per QLinearConv launch of the program, in program order: the algorithmic work that prices it against
    the two roofs.  ops = 2 * MACs.  bytes = what the launch must move at least: the input pixels it needs (a 1x1
    convolution with stride s reads every s-th pixel of every s-th row only), the weights, the output, and with
    `fuse_residual` the residual operand of the Add(+Relu) group behind it (whose sum is then the output).  With
    `pair_convs` two convolutions of one value are one launch (pair_convolutions): the input counts once.  All tensors
    are 8-bit.  A launch belongs to the roof that takes longer at the published peaks."""
    convs, shapes = model["convs"], model["shapes"]
    prog = pair_convolutions(model["program"], convs) if pair_convs else model["program"]
    rows = []
    for i, ins in enumerate(prog):
        if ins[0] not in ("QLinearConv", "QLinearConvPair"):
            continue
        c = convs[ins[3]]
        n, cin, h, w = shapes[ins[2]]
        _, oc, oh, ow = shapes[ins[1]]
        k = c.wq.shape[2]
        x_bytes = n * cin * (oh * ow if k == 1 else h * w)
        nbytes = x_bytes + c.wq.size + n * oc * oh * ow
        ops = 2.0 * c.macs(shapes[ins[1]])
        name = c.name
        if ins[0] == "QLinearConvPair":
            c2 = convs[ins[5]]
            oc2 = shapes[ins[4]][1]
            nbytes += c2.wq.size + n * oc2 * oh * ow
            ops += 2.0 * c2.macs(shapes[ins[4]])
            oc += oc2
            name += "+" + c2.name
        residual = False
        if ins[0] == "QLinearConv" and fuse_residual and i + 1 < len(prog) and prog[i + 1][0] in ("AddRelu", "Add") and ins[1] in prog[i + 1][2:4]:
            # the group is computed in this launch when the convolution result has no other reader
            readers = [j for j in prog if ins[1] in j[2:]]
            if len(readers) == 1:
                residual = True
                nbytes += n * oc * oh * ow
        rows.append(dict(name=name, cin=cin, cout=oc, k=k, stride=c.stride, group=c.group, out_hw=oh, ops=ops,
                         bytes=float(nbytes), residual=residual))
    return rows


def run_reference(model, orc, x, keep=None):
    """Executes the program with a CPU executor `orc` that offers the oracle's functions
    (quantize_linear, qlinear_conv_int, max_pool_q8, ...).  Test and benchmark code passes
    the oracle module in; this module itself never imports it."""
    q = model["qparams"]
    v = {"x": x}
    for ins in model["program"]:
        kind, out = ins[0], ins[1]
        if kind == "QuantizeLinear":
            v[out] = orc.quantize_linear(v[ins[2]], ins[3], ins[4], np.uint8)
        elif kind == "QLinearConv":
            c = model["convs"][ins[3]]
            v[out] = orc.qlinear_conv_int(v[ins[2]], c.x_scale, c.x_zp, c.wq, c.w_scale, c.w_zp, c.y_scale, c.y_zp,
                                          np.uint8, bias=c.bias_q, strides=(c.stride, c.stride), pads=(c.pad, c.pad),
                                          group=c.group, bias_mode=orc.BIAS_ONNX_INT32)
        elif kind == "MaxPool":
            v[out] = orc.max_pool_q8(v[ins[2]], (ins[3], ins[3]), (ins[4], ins[4]), (ins[5], ins[5]), ins[6])
        elif kind == "AddRelu":
            a = orc.dequantize_linear(v[ins[2]], *q[ins[2]])
            b = orc.dequantize_linear(v[ins[3]], *q[ins[3]])
            v[out] = orc.quantize_linear(orc.relu(orc.binary(orc.ADD, a, b)), q[out][0], q[out][1], np.uint8)
        elif kind == "Add":
            a = orc.dequantize_linear(v[ins[2]], *q[ins[2]])
            b = orc.dequantize_linear(v[ins[3]], *q[ins[3]])
            v[out] = orc.quantize_linear(orc.binary(orc.ADD, a, b), q[out][0], q[out][1], np.uint8)
        elif kind == "AveragePool":
            v[out] = orc.average_pool_q8(v[ins[2]], q[ins[2]][0], q[ins[2]][1], (ins[3], ins[3]), (1, 1), (0, 0),
                                         q[out][0], q[out][1], np.uint8)
        elif kind == "DequantizeLinear":
            v[out] = orc.dequantize_linear(v[ins[2]], ins[3], ins[4])
        else:
            raise ValueError(kind)
        if keep is not None:
            for name in list(v):
                if name not in keep and name != out and not _still_needed(model["program"], ins, name):
                    del v[name]
    return v


def _still_needed(program, current, name):
    seen = False
    for ins in program:
        if ins is current:
            seen = True
            continue
        if seen and name in ins[2:]:
            return True
    return False
