"""Seeded builders of the benchmark configurations as post-LPT graphs.

The reference ships no whole-model builders or weights, so the networks are defined here:
architecture, He-normal weights (BatchNorm folded into conv + bias), a seeded calibration batch
run in fp32 on the host to fix every activation FakeQuantize range, and then the graph that the
stock low-precision transformations leave for a plugin (derivation in ``QuantizedNet``).
"""
import numpy as np

from . import lpt
from .graph import Graph
from .tensor import F32, I8, U8


class QuantizedNet:
    """Emits post-LPT layers.  An *activation* is a dict(node=<u8 value id>, scale=<f32 scalar>):
    the u8 FakeQuantize output and the scale of its pending dequantization Multiply
    (decomposeFakeQuantize: scale = (out_high - out_low) / 255 for [0, ih] ranges).

    Per layer, with s[c] = s_act * s_w[c] (ConvolutionTransformation, optimizeMultipliesAfter):
        Conv'(u8 x, i8 W) -> Add(b[c] / s[c])  (AddTransformation / swapMultiplyAndAdd)
        followed either by the next activation FakeQuantize with the Multiply folded into its
        input range (FakeQuantizeTransformation::fuseElementwise: il / s[c], ih / s[c]), or by
        Multiply(s[c]) when the value is used in f32 (residual Add, graph output).
    ReLU in front of a FakeQuantize with input_low >= 0 is already gone before LPT
    (ReluFakeQuantizeFusion), so it only survives in f32 tails.
    """

    def __init__(self):
        self.g = Graph()

    # -- graph input ---------------------------------------------------------------------------
    def input(self, name, shape, in_high, u8=False):
        """f32 graph input, or (u8=True) a u8 one behind a Convert to f32: what a plugin sees when the user
        sets input precision U8 (benchmark_app's default for images)."""
        g = self.g
        x = g.convert(g.parameter(name, shape, U8), F32) if u8 else g.parameter(name, shape)
        d = lpt.decompose_fake_quantize(256, np.float32(0), np.float32(in_high))
        q = g.fake_quantize(x, np.float32(0), np.float32(in_high), d["new_low"], d["new_high"], 256, U8)
        return dict(node=q, scale=np.float32(d["scale"]))

    def _channel(self, v, rank):
        v = np.asarray(v, np.float32)
        return v.reshape((1, -1) + (1,) * (rank - 2))

    def asymmetric(self, y, lo, hi):
        """Activation FakeQuantize with an asymmetric range [lo, hi]: u8 levels 0 .. 255 with a zero point.
        The activation carries the exact f32 shift (for f32 consumers) and the integer zero point that
        ConvolutionTransformation leaves as Subtract in front of a convolution."""
        d = lpt.decompose_fake_quantize(256, np.float32(lo), np.float32(hi), allow_zero_point=True)
        assert d["has_zero_point"] and d["precision"] == U8
        q = self.g.fake_quantize(y, np.float32(lo), np.float32(hi), d["new_low"], d["new_high"], 256, U8)
        return dict(node=q, scale=np.float32(d["scale"]), shift=np.float32(d["shift"]),
                    zero_point=np.float32(lpt.round_zero_point(d["shift"])))

    def asymmetric_per_channel(self, y, lo, hi):
        """The same with one interval per channel (allowed in front of a GroupConvolution, whose per-channel
        dequantization folds into its per-channel weights scales): scales, shifts and zero points are vectors."""
        d = [lpt.decompose_fake_quantize(256, np.float32(a), np.float32(b), allow_zero_point=True) for a, b in zip(lo, hi)]
        assert all(k["precision"] == U8 for k in d) and len({(k["new_low"], k["new_high"]) for k in d}) == 1
        rank = 4
        q = self.g.fake_quantize(y, self._channel(np.asarray(lo, np.float32), rank), self._channel(np.asarray(hi, np.float32), rank),
                                 d[0]["new_low"], d[0]["new_high"], 256, U8)
        return dict(node=q, scale=np.array([k["scale"] for k in d], np.float32).reshape(-1),
                    shift=np.array([k["shift"] for k in d], np.float32).reshape(-1),
                    zero_point=np.array([lpt.round_zero_point(k["shift"]) for k in d], np.float32).reshape(-1))

    def _accumulate(self, act, w, bias, conv_attrs, matmul=False):
        """[Subtract(zero point)] -> Conv'/MatMul' -> Add(b / s): returns (node, s[c])."""
        g = self.g
        wq, s_w = lpt.quantize_weights(w, 255)
        groups = conv_attrs.pop("groups", 0)
        s_a = np.asarray(act["scale"], np.float32).reshape(-1)
        if s_a.size > 1 and s_a.size != s_w.size:
            # per-channel activation scales in front of a grouped convolution: one scale per group (the transformation
            # takes the layer only if the scales are equal inside every group, group_convolution.cpp via
            # WeightableLayerTransformation::canBeTransformed), repeated over the group's output channels
            G = groups or s_a.size
            per_group = s_a.reshape(G, -1)
            assert np.all(per_group == per_group[:, :1])
            s_a = np.repeat(per_group[:, 0], s_w.size // G)
        s = (s_a * s_w).astype(np.float32)                                 # fold<Multiply>(s_a, s_w)
        out_rank = 2 if matmul else w.ndim          # [N, C, H, W], or [N, C, W] for filters over one spatial dimension
        if groups:
            # [OC, IC / G, kh, kw] -> [G, OC / G, IC / G, kh, kw]
            wq = wq.reshape((groups, wq.shape[0] // groups) + wq.shape[1:])
            conv_attrs["grouped"] = True
        elif conv_attrs.get("grouped"):
            # GroupConvolution weights: FQ on [C, 1, kh, kw] then Reshape to [G, 1, 1, kh, kw]
            # (the pattern LPT recognises, group_convolution.cpp:50-52); both fold into one constant
            wq = wq.reshape((wq.shape[0], 1, 1) + wq.shape[2:])
        wc = g.constant(wq, I8)
        x = act["node"]
        zp = np.asarray(act.get("zero_point", 0), np.float32)
        if np.any(zp != 0):                    # TypeRelaxed Subtract(u8, u8) -> f32, written as Convert + Subtract
            x = g.subtract(g.convert(x, F32), g.constant(zp.reshape(()) if zp.ndim == 0 else self._channel(zp, out_rank)))
        rank = out_rank
        if matmul:
            y = g.matmul(x, wc, False, True)
        else:
            y = g.convolution(x, wc, **conv_attrs)
        if bias is not None:
            bdiv = lpt.swap_multiply_and_add(bias, s)                          # bi / ai
            y = g.add(y, g.constant(self._channel(bdiv, rank)))
        return y, s, rank

    @staticmethod
    def signed_range(m):
        """FakeQuantize range that getPrecisionDetails resolves to i8 without a zero point."""
        hi = np.float32(m)
        return np.float32(-hi * np.float32(128.0) / np.float32(127.0)), hi

    def conv(self, act, w, bias, out_high, strides=(1, 1), pads=(0, 0), dilations=(1, 1), signed=False,
             grouped=False, groups=0):
        """Quantized conv feeding the next activation FakeQuantize: [0, out_high] -> u8 (ReLU fused
        away) or, for linear outputs, the symmetric range of signed_range(out_high) -> i8."""
        g = self.g
        attrs = dict(strides=strides, dilations=dilations, pads_begin=pads, pads_end=pads, grouped=grouped)
        if groups:
            attrs["groups"] = groups
        y, s, rank = self._accumulate(act, w, bias, attrs)
        lo, hi = self.signed_range(out_high) if signed else (np.float32(0), np.float32(out_high))
        d = lpt.decompose_fake_quantize(256, lo, hi)
        il, ih = lpt.fuse_elementwise(lpt.MULTIPLY, lo, hi, s)             # fold<Divide>(il, s), fold<Divide>(ih, s)
        q = g.fake_quantize(y, self._channel(il, rank), self._channel(ih, rank), d["new_low"], d["new_high"],
                            256, d["precision"])
        return dict(node=q, scale=np.float32(d["scale"]))

    def conv_relu6(self, act, w, bias, out_high, strides=(1, 1), pads=(0, 0), grouped=False):
        """Conv -> bias -> ReLU6 -> FakeQuantize [0, out_high].  The dequantization Multiply is per
        channel, so ClampTransformation leaves the Clamp in f32 (clamp.cpp:100-112) and the
        FakeQuantize keeps its per-tensor range."""
        g = self.g
        attrs = dict(strides=strides, dilations=(1, 1), pads_begin=pads, pads_end=pads, grouped=grouped)
        y, s, rank = self._accumulate(act, w, bias, attrs)
        y = g.clamp(g.multiply(y, g.constant(self._channel(s, rank))), 0.0, 6.0)
        return self.requantize(y, out_high)

    def conv_f32(self, act, w, bias, strides=(1, 1), pads=(0, 0), relu=False, matmul=False, grouped=False, groups=0):
        """Quantized conv / FC whose result is consumed in f32: ... -> Multiply(s[c]) [-> ReLU]."""
        g = self.g
        attrs = dict(strides=strides, dilations=(1,) * len(strides), pads_begin=pads, pads_end=pads)
        if grouped:
            attrs["grouped"] = True
        if groups:
            attrs["groups"] = groups
        y, s, rank = self._accumulate(act, w, bias, attrs, matmul)
        y = g.multiply(y, g.constant(self._channel(s, rank)))
        return g.relu(y) if relu else y

    def dequantize(self, act):
        """Convert + Multiply left on a u8 value that is consumed in f32."""
        g = self.g
        return g.multiply(g.convert(act["node"], F32), g.constant(np.float32(act["scale"]).reshape(())))

    def requantize(self, y, out_high, signed=False):
        """Activation FakeQuantize on an f32 value (no pending Multiply to fold)."""
        lo, hi = self.signed_range(out_high) if signed else (np.float32(0), np.float32(out_high))
        d = lpt.decompose_fake_quantize(256, lo, hi)
        q = self.g.fake_quantize(y, lo, hi, d["new_low"], d["new_high"], 256, d["precision"])
        return dict(node=q, scale=np.float32(d["scale"]))

    def max_pool(self, act, kernel, strides, pads):
        # MaxPoolTransformation: the Multiply moves behind the pool, which then runs on u8
        return dict(node=self.g.max_pool(act["node"], kernel, strides, pads, pads), scale=act["scale"])


# ---------------------------------------------------------------------------------------------
def he_normal(rng, shape):
    fan_in = int(np.prod(shape[1:]))
    return (rng.standard_normal(shape, dtype=np.float32) * np.float32(np.sqrt(2.0 / fan_in))).astype(np.float32)


def conv_block(seed=20211, n=1, c=64, hw=56, oc=64, u8_input=False):
    """benchmark configuration 1: FQ(u8) -> Conv 3x3 s1 p1 (per-channel i8 weights) -> bias -> ReLU, f32 out.
    u8_input: the graph input is a u8 tensor (values 0 .. 255) behind a Convert to f32."""
    rng = np.random.default_rng(seed)
    x = rng.integers(0, 256, (n, c, hw, hw)).astype(np.uint8) if u8_input else \
        rng.uniform(0, 2.55, (n, c, hw, hw)).astype(np.float32)
    w = (rng.standard_normal((oc, c, 3, 3), dtype=np.float32) * np.float32(0.05)).astype(np.float32)
    b = (rng.standard_normal(oc, dtype=np.float32) * np.float32(0.1)).astype(np.float32)
    net = QuantizedNet()
    a = net.input("data", x.shape, 255.0, u8=True) if u8_input else net.input("data", x.shape, 2.55)
    y = net.conv_f32(a, w, b, pads=(1, 1), relu=True)
    net.g.result(y, "out")
    return net.g, dict(data=x), dict(w=w, b=b)


RESNET50_STAGES = [(64, 3, 1), (128, 4, 2), (256, 6, 2), (512, 3, 2)]


def resnet50_weights(seed=20211, classes=1000, width=64, stages=RESNET50_STAGES):
    """ResNet-50 v1.5 parameters: He-normal convs with a folded-BN bias ~ N(0, 0.1)."""
    rng = np.random.default_rng(seed)
    P = {}

    def conv(name, oc, ic, k):
        P[name + ".w"] = he_normal(rng, (oc, ic, k, k))
        P[name + ".b"] = (rng.standard_normal(oc, dtype=np.float32) * np.float32(0.1)).astype(np.float32)

    conv("conv1", width, 3, 7)
    ic = width
    for si, (mid, blocks, _) in enumerate(stages):
        mid = mid * width // 64
        for bi in range(blocks):
            p = "layer%d.%d" % (si + 1, bi)
            conv(p + ".a", mid, ic, 1)
            conv(p + ".b", mid, mid, 3)
            conv(p + ".c", mid * 4, mid, 1)
            if bi == 0:
                conv(p + ".ds", mid * 4, ic, 1)
            ic = mid * 4
    P["fc.w"] = he_normal(rng, (classes, ic))
    P["fc.b"] = (rng.standard_normal(classes, dtype=np.float32) * np.float32(0.1)).astype(np.float32)
    return P


def resnet50_fp32(P, x, stages=RESNET50_STAGES, record=None):
    """fp32 forward on the host (torch CPU) — used only to calibrate activation ranges."""
    import torch
    import torch.nn.functional as F

    def t(a):
        return torch.from_numpy(np.ascontiguousarray(a))

    def conv(name, v, stride=1, pad=0):
        return F.conv2d(v, t(P[name + ".w"]), t(P[name + ".b"]), stride=stride, padding=pad)

    def rec(name, v):
        if record is not None:
            record[name] = max(record.get(name, 0.0), float(v.max()))
        return v

    with torch.no_grad():
        v = rec("input", t(x))
        v = rec("conv1", F.relu(conv("conv1", v, 2, 3)))
        v = F.max_pool2d(v, 3, 2, 1)
        for si, (_, blocks, stride) in enumerate(stages):
            for bi in range(blocks):
                p = "layer%d.%d" % (si + 1, bi)
                s = stride if bi == 0 else 1
                y = rec(p + ".a", F.relu(conv(p + ".a", v)))
                y = rec(p + ".b", F.relu(conv(p + ".b", y, s, 1)))      # v1.5: stride on the 3x3
                y = conv(p + ".c", y)
                sc = conv(p + ".ds", v, s) if bi == 0 else v
                v = rec(p + ".out", F.relu(y + sc))
        v = rec("pool", v.mean(dim=(2, 3)))
        v = F.linear(v, t(P["fc.w"]), t(P["fc.b"]))
    return v.numpy()


def resnet50(batch=1, res=224, seed=20211, classes=1000, width=64, stages=RESNET50_STAGES, calib_batch=2, u8_input=False):
    """benchmark configuration 3 as a post-LPT graph.  Returns (graph, meta) where meta holds the
    parameters, the calibrated ranges and the ids of every quantized activation.
    u8_input: the graph input is a u8 image (values 0 .. 255, input precision U8 as benchmark_app sets it for image
    inputs) behind a Convert; the first layer's weights are those of a model fed 0 .. 255 instead of 0 .. 1."""
    P = resnet50_weights(seed, classes, width, stages)
    rng = np.random.default_rng(seed + 1)
    calib = rng.uniform(0, 1, (calib_batch, 3, res, res)).astype(np.float32)
    if u8_input:
        P["conv1.w"] = (P["conv1.w"] / np.float32(255)).astype(np.float32)
        calib = np.floor(calib * np.float32(256)).clip(0, 255).astype(np.float32)
    R = {}
    resnet50_fp32(P, calib, stages, R)
    if u8_input:
        R["input"] = 255.0                      # every byte is its own level
    net = QuantizedNet()
    g = net.g
    acts = {}
    a = net.input("data", (batch, 3, res, res), R["input"], u8=u8_input)
    acts["input"] = a
    a = net.conv(a, P["conv1.w"], P["conv1.b"], R["conv1"], strides=(2, 2), pads=(3, 3))
    acts["conv1"] = a
    a = net.max_pool(a, (3, 3), (2, 2), (1, 1))
    acts["maxpool"] = a
    for si, (_, blocks, stride) in enumerate(stages):
        for bi in range(blocks):
            p = "layer%d.%d" % (si + 1, bi)
            s = stride if bi == 0 else 1
            ya = net.conv(a, P[p + ".a.w"], P[p + ".a.b"], R[p + ".a"])
            yb = net.conv(ya, P[p + ".b.w"], P[p + ".b.b"], R[p + ".b"], strides=(s, s), pads=(1, 1))
            yc = net.conv_f32(yb, P[p + ".c.w"], P[p + ".c.b"])
            if bi == 0:
                sc = net.conv_f32(a, P[p + ".ds.w"], P[p + ".ds.b"], strides=(s, s))
            else:
                sc = net.dequantize(a)
            # the residual Add stays f32 (AddTransformation leaves it: the conv branch is not low
            # precision); the ReLU behind it was fused into the next FakeQuantize before LPT
            a = net.requantize(g.add(yc, sc), R[p + ".out"])
            acts[p + ".a"], acts[p + ".b"], acts[p + ".out"] = ya, yb, a
    final_hw = res // (4 * int(np.prod([st[2] for st in stages])))     # stem and max-pool halve twice, then the stages' strides
    y = g.avg_pool(a["node"], (final_hw, final_hw), (1, 1), (0, 0), (0, 0), exclude_pad=True, out_dtype=F32)
    y = g.reshape(y, (batch, P["fc.w"].shape[1]))
    d = lpt.decompose_fake_quantize(256, np.float32(0), np.float32(R["pool"]))
    s_x = np.float32(a["scale"])
    il, ih = lpt.fuse_elementwise(lpt.MULTIPLY, np.float32(0), np.float32(R["pool"]), s_x)
    q = g.fake_quantize(y, il.reshape(()), ih.reshape(()), d["new_low"], d["new_high"], 256, U8)
    pooled = dict(node=q, scale=np.float32(d["scale"]))
    acts["pool"] = pooled
    logits = net.conv_f32(pooled, P["fc.w"], P["fc.b"], matmul=True)
    g.result(logits, "logits")
    macs = resnet50_macs(res, classes, width, stages)
    return g, dict(params=P, ranges=R, acts=acts, macs_per_image=macs, calib=calib)


def resnet50_macs(res=224, classes=1000, width=64, stages=RESNET50_STAGES):
    h = res // 2
    macs = h * h * width * 3 * 49
    h = h // 2
    ic = width
    for mid, blocks, stride in stages:
        mid = mid * width // 64
        for bi in range(blocks):
            s = stride if bi == 0 else 1
            macs += h * h * mid * ic
            h2 = h // s
            macs += h2 * h2 * mid * mid * 9
            macs += h2 * h2 * mid * 4 * mid
            if bi == 0:
                macs += h2 * h2 * mid * 4 * ic
            ic = mid * 4
            h = h2
    return macs + classes * ic


# ---------------------------------------------------------------------------------------------
MOBILENETV2_BLOCKS = [(1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 3, 2), (6, 64, 4, 2), (6, 96, 3, 1), (6, 160, 3, 2),
                      (6, 320, 1, 1)]


def _mbv2_layers(width=1.0, blocks=MOBILENETV2_BLOCKS, last=1280):
    """(name, kind, ic, oc, stride, residual) in execution order; channels rounded to multiples of 8."""
    def ch(c):
        return max(8, int(round(c * width / 8.0)) * 8)
    layers = [("stem", "conv3", 3, ch(32), 2, False)]
    ic = ch(32)
    for bi, (t, c, n, s) in enumerate(blocks):
        oc = ch(c)
        for i in range(n):
            p = "b%d.%d" % (bi, i)
            mid = ic * t
            stride = s if i == 0 else 1
            if t != 1:
                layers.append((p + ".expand", "pw_relu6", ic, mid, 1, False))
            layers.append((p + ".dw", "dw", mid, mid, stride, False))
            layers.append((p + ".project", "pw_linear", mid, oc, 1, stride == 1 and ic == oc))
            ic = oc
    layers.append(("head", "pw_relu6", ic, ch(last), 1, False))
    return layers


def mobilenet_v2_weights(seed=20211, classes=1000, width=1.0, blocks=MOBILENETV2_BLOCKS, last=1280):
    rng = np.random.default_rng(seed)
    P = {}
    for name, kind, ic, oc, _, _ in _mbv2_layers(width, blocks, last):
        shape = (oc, 1, 3, 3) if kind == "dw" else (oc, ic, 3, 3) if kind == "conv3" else (oc, ic, 1, 1)
        P[name + ".w"] = he_normal(rng, shape)
        P[name + ".b"] = (rng.standard_normal(oc, dtype=np.float32) * np.float32(0.1)).astype(np.float32)
    feat = _mbv2_layers(width, blocks, last)[-1][3]
    P["fc.w"] = he_normal(rng, (classes, feat))
    P["fc.b"] = (rng.standard_normal(classes, dtype=np.float32) * np.float32(0.1)).astype(np.float32)
    return P


def mobilenet_v2_fp32(P, x, width=1.0, blocks=MOBILENETV2_BLOCKS, last=1280, record=None):
    """fp32 forward on the host (torch CPU) for calibration."""
    import torch
    import torch.nn.functional as F

    def t(a):
        return torch.from_numpy(np.ascontiguousarray(a))

    def rec(name, v, signed=False):
        if record is not None:
            record[name] = max(record.get(name, 0.0), float(v.abs().max() if signed else v.max()))
        return v

    names = {n for n, *_ in _mbv2_layers(width, blocks, last)}
    with torch.no_grad():
        v = rec("input", t(x))
        block_in = None
        for name, kind, ic, oc, stride, residual in _mbv2_layers(width, blocks, last):
            w, b = t(P[name + ".w"]), t(P[name + ".b"])
            if name.endswith(".expand") or (kind == "dw" and name[:-3] + ".expand" not in names):
                block_in = v
            if kind == "conv3":
                v = rec(name, F.relu6(F.conv2d(v, w, b, stride=stride, padding=1)))
            elif kind == "pw_relu6":
                v = rec(name, F.relu6(F.conv2d(v, w, b)))
            elif kind == "dw":
                v = rec(name, F.relu6(F.conv2d(v, w, b, stride=stride, padding=1, groups=oc)))
            else:
                v = F.conv2d(v, w, b)
                if residual:
                    v = v + block_in
                v = rec(name, v, signed=True)
        v = rec("pool", v.mean(dim=(2, 3)))
        v = F.linear(v, t(P["fc.w"]), t(P["fc.b"]))
    return v.numpy()


def mobilenet_v2(batch=1, res=224, seed=20211, classes=1000, width=1.0, blocks=MOBILENETV2_BLOCKS, last=1280,
                 calib_batch=2):
    """benchmark configuration 4 as a post-LPT graph: ReLU6 outputs are u8 [0, max], linear bottleneck
    outputs symmetric i8; depthwise layers are GroupConvolutions with [G,1,1,3,3] i8 filters."""
    P = mobilenet_v2_weights(seed, classes, width, blocks, last)
    rng = np.random.default_rng(seed + 1)
    calib = rng.uniform(0, 1, (calib_batch, 3, res, res)).astype(np.float32)
    R = {}
    mobilenet_v2_fp32(P, calib, width, blocks, last, R)
    net = QuantizedNet()
    g = net.g
    acts = {}
    a = net.input("data", (batch, 3, res, res), R["input"])
    layers = _mbv2_layers(width, blocks, last)
    names = {n for n, *_ in layers}
    block_in = None
    macs = 0
    hw = res
    for name, kind, ic, oc, stride, residual in layers:
        w, b = P[name + ".w"], P[name + ".b"]
        if name.endswith(".expand") or (kind == "dw" and name[:-3] + ".expand" not in names):
            block_in = a
        if kind == "conv3":
            a = net.conv_relu6(a, w, b, R[name], strides=(stride, stride), pads=(1, 1))
            hw //= stride
            macs += hw * hw * oc * ic * 9
        elif kind == "pw_relu6":
            a = net.conv_relu6(a, w, b, R[name])
            macs += hw * hw * oc * ic
        elif kind == "dw":
            a = net.conv_relu6(a, w, b, R[name], strides=(stride, stride), pads=(1, 1), grouped=True)
            hw //= stride
            macs += hw * hw * oc * 9
        else:
            macs += hw * hw * oc * ic
            if residual:
                y = net.conv_f32(a, w, b)
                a = net.requantize(g.add(y, net.dequantize(block_in)), R[name], signed=True)
            else:
                a = net.conv(a, w, b, R[name], signed=True)
        acts[name] = a
    y = g.avg_pool(a["node"], (hw, hw), (1, 1), (0, 0), (0, 0), exclude_pad=True, out_dtype=F32)
    y = g.reshape(y, (batch, P["fc.w"].shape[1]))
    d = lpt.decompose_fake_quantize(256, np.float32(0), np.float32(R["pool"]))
    s_x = np.float32(a["scale"])
    il, ih = lpt.fuse_elementwise(lpt.MULTIPLY, np.float32(0), np.float32(R["pool"]), s_x)
    q = g.fake_quantize(y, il.reshape(()), ih.reshape(()), d["new_low"], d["new_high"], 256, U8)
    pooled = dict(node=q, scale=np.float32(d["scale"]))
    acts["pool"] = pooled
    logits = net.conv_f32(pooled, P["fc.w"], P["fc.b"], matmul=True)
    g.result(logits, "logits")
    macs += P["fc.w"].size
    return g, dict(params=P, ranges=R, acts=acts, macs_per_image=macs, calib=calib)


# ---------------------------------------------------------------------------------------------
BERT_RANGES = dict(x=4.0, q=1.2, k=3.0, v=3.0, p=1.0, ctx=1.0, h1=4.0, g=3.0)


def bert_encoder(layers=12, hidden=768, heads=12, ffn=3072, batch=16, seq=384, seed=20211, ranges=None, vocab=0,
                 mask=False, unsigned_probs=False):
    """benchmark configuration 5: BERT-base style encoder stack in its post-LPT form.  Activations are
    per-tensor symmetric i8 (FakeQuantize ranges of signed_range), weights per-channel i8, Softmax /
    LayerNorm (MVN, Multiply, Add) / Gelu stay f32.

    Per layer, with x the f32 hidden states [batch, seq, hidden]:
        xq = FQ(x);  q, k, v = FQ(MatMul'(xq, W^T) + b')        dequantization folded into the FQ range
        s = MatMul'(heads(q), heads(k)^T) * (s_q s_k);  p = Softmax(s)   1/sqrt(d) folded into W_q
        c = merge(MatMul'(FQ(p), heads(v)) * (s_p s_v))
        a = (MatMul'(FQ(c), W_o^T) + b') * s + x;  h1 = LayerNorm(a)
        f = Gelu((MatMul'(FQ(h1), W_1^T) + b') * s)
        o = (MatMul'(FQ(f), W_2^T) + b') * s + h1;  y = LayerNorm(o)
    (MatMulTransformation, mat_mul.cpp:81-171; AddTransformation moves the bias in front of the
    Multiply, add.cpp:125-153; FakeQuantizeTransformation::fuseElementwise, fake_quantize.cpp:127-157.)

    vocab > 0 puts the embedding front end in front (the graph input is then the i32 token ids
    [batch, seq] instead of the f32 hidden states): Gather(word table [vocab, hidden], ids) +
    position table [seq, hidden] + token-type row [hidden], LayerNorm.

    mask=True adds a second graph input "attention_mask" f32 [batch, 1, 1, seq] that is added to the
    scaled scores of every layer in front of the Softmax (0 for tokens to attend to, -10000 for padding).

    Returns (graph, meta); meta["layers"][l] maps tensor names to node ids, meta["glue"] lists the
    nodes that only have tolerance parity (Softmax, LayerNorm tails, Gelu)."""
    assert hidden % heads == 0
    D = hidden // heads
    r = dict(BERT_RANGES)
    r.update(ranges or {})
    rng = np.random.default_rng(seed)
    net = QuantizedNet()
    g = net.g
    nrm = lambda *shape: (rng.standard_normal(shape, dtype=np.float32) * np.float32(0.02)).astype(np.float32)
    meta = dict(layers=[], glue=[], macs=0, linear=[], norm=[])   # linear / norm: the float parameters in the order of their use
    if vocab:
        from .tensor import I32
        ids = g.parameter("input_ids", (batch, seq), I32)
        emb = g.gather(g.constant(nrm(vocab, hidden)), ids, 0)
        emb = g.add(g.add(emb, g.constant(nrm(seq, hidden))), g.constant(nrm(hidden)))
        meta["embeddings"] = emb
    else:
        x = g.parameter("hidden_states", (batch, seq, hidden))

    def fq(v, absmax):
        lo, hi = net.signed_range(absmax)
        d = lpt.decompose_fake_quantize(256, lo, hi)
        assert d["precision"] == I8
        return dict(node=g.fake_quantize(v, lo, hi, d["new_low"], d["new_high"], 256, I8), scale=np.float32(d["scale"]))

    def fq_u8(v, high):
        """FakeQuantize of a non-negative value (Softmax output) to u8 levels 0..255"""
        from .tensor import U8
        d = lpt.decompose_fake_quantize(256, np.float32(0), np.float32(high))
        assert d["precision"] == U8 and d["shift"] == 0
        return dict(node=g.fake_quantize(v, np.float32(0), np.float32(high), d["new_low"], d["new_high"], 256, U8),
                    scale=np.float32(d["scale"]))

    def linear(act, w, b):
        """MatMul' -> Add(b / s): returns (node, s[c])"""
        wq, s_w = lpt.quantize_weights(w, 255)
        s = (np.float32(act["scale"]) * s_w).astype(np.float32)
        meta["linear"].append((w, b))
        y = g.matmul(act["node"], g.constant(wq, I8), False, True)
        return g.add(y, g.constant(lpt.swap_multiply_and_add(b, s))), s

    def linear_fq(act, w, b, absmax):
        y, s = linear(act, w, b)
        lo, hi = net.signed_range(absmax)
        d = lpt.decompose_fake_quantize(256, lo, hi)
        il, ih = lpt.fuse_elementwise(lpt.MULTIPLY, lo, hi, s)
        q = g.fake_quantize(y, il, ih, d["new_low"], d["new_high"],
                            256, I8)
        return dict(node=q, scale=np.float32(d["scale"]))

    def linear_f32(act, w, b):
        y, s = linear(act, w, b)
        return g.multiply(y, g.constant(s))

    def layer_norm(v):
        n = g.mvn(v, (-1,), True, 1e-5, True)
        gamma, beta = np.float32(1) + nrm(hidden), nrm(hidden)
        meta["norm"].append((gamma, beta))
        out = g.add(g.multiply(n, g.constant(gamma)), g.constant(beta))
        meta["glue"].append(out)
        return out

    def split_heads(node):
        return g.transpose(g.reshape(node, (batch, seq, heads, D)), (0, 2, 1, 3))

    if vocab:
        x = layer_norm(emb)
        meta["embedding_norm"] = x
    mask_node = g.parameter("attention_mask", (batch, 1, 1, seq)) if mask else None
    for _ in range(layers):
        L = {}
        wq_ = nrm(hidden, hidden) * np.float32(1.0 / np.sqrt(D))
        xq = fq(x, r["x"])
        q = linear_fq(xq, wq_, nrm(hidden), r["q"])
        k = linear_fq(xq, nrm(hidden, hidden), nrm(hidden), r["k"])
        v = linear_fq(xq, nrm(hidden, hidden), nrm(hidden), r["v"])
        s = g.multiply(g.matmul(split_heads(q["node"]), split_heads(k["node"]), False, True),
                       g.constant(np.float32(q["scale"] * k["scale"]).reshape(())))
        if mask_node is not None:
            s = g.add(s, mask_node)
        p = g.softmax(s, -1)
        meta["glue"].append(p)
        pq = fq_u8(p, r["p"]) if unsigned_probs else fq(p, r["p"])
        c = g.multiply(g.matmul(pq["node"], split_heads(v["node"])),
                       g.constant(np.float32(pq["scale"] * v["scale"]).reshape(())))
        c_t = g.transpose(c, (0, 2, 1, 3))
        c_m = g.reshape(c_t, (batch, seq, hidden))
        cq = fq(c_m, r["ctx"])
        a = g.add(linear_f32(cq, nrm(hidden, hidden), nrm(hidden)), x)
        h1 = layer_norm(a)
        h1q = fq(h1, r["h1"])
        f = linear_f32(h1q, nrm(ffn, hidden), nrm(ffn))
        gl = g.gelu(f)
        meta["glue"].append(gl)
        gq = fq(gl, r["g"])
        o = g.add(linear_f32(gq, nrm(hidden, ffn), nrm(hidden)), h1)
        y = layer_norm(o)
        L.update(xq=xq["node"], q=q["node"], k=k["node"], v=v["node"], scores=s, p=p, pq=pq["node"], ctx=c_t,
                 ctxq=cq["node"], attn=a, h1=h1, h1q=h1q["node"], up=f, gelu=gl, gq=gq["node"], down=o, y=y)
        meta["layers"].append(L)
        x = y
    g.result(x, "out")
    T = batch * seq
    meta["macs"] = layers * (T * (4 * hidden * hidden + 2 * hidden * ffn) + 2 * batch * heads * seq * seq * D)
    return g, meta


def zero_point_net(seed=31, n=2, c=32, hw=20, oc=(48, 32)):
    """Two quantized convolutions whose inputs have asymmetric ranges (u8 with zero points): a padded,
    strided 3x3 and a 1x1; the second one's input FakeQuantize (asymmetric as well) rides in the first
    one's epilogue.  Returns (graph, feeds, meta)."""
    rng = np.random.default_rng(seed)
    x = rng.normal(0.4, 1.0, (n, c, hw, hw)).astype(np.float32)
    net = QuantizedNet()
    g = net.g
    a0 = net.asymmetric(g.parameter("data", x.shape), -1.7, 2.9)
    w1 = (rng.standard_normal((oc[0], c, 3, 3), dtype=np.float32) * np.float32(0.06)).astype(np.float32)
    b1 = (rng.standard_normal(oc[0], dtype=np.float32) * np.float32(0.2)).astype(np.float32)
    y1, s1, rank = net._accumulate(a0, w1, b1, dict(strides=(2, 2), dilations=(1, 1), pads_begin=(1, 1), pads_end=(1, 1)))
    lo, hi = np.float32(-2.2), np.float32(1.4)
    d = lpt.decompose_fake_quantize(256, lo, hi, allow_zero_point=True)
    q1 = g.fake_quantize(y1, net._channel((lo / s1).astype(np.float32), rank), net._channel((hi / s1).astype(np.float32), rank),
                         d["new_low"], d["new_high"], 256, U8)
    a1 = dict(node=q1, scale=np.float32(d["scale"]), shift=np.float32(d["shift"]),
              zero_point=np.float32(lpt.round_zero_point(d["shift"])))
    w2 = (rng.standard_normal((oc[1], oc[0], 1, 1), dtype=np.float32) * np.float32(0.1)).astype(np.float32)
    b2 = (rng.standard_normal(oc[1], dtype=np.float32) * np.float32(0.2)).astype(np.float32)
    y2 = net.conv_f32(a1, w2, b2)
    g.result(y2, "out")
    return g, dict(data=x), dict(acts=dict(a0=a0, a1=a1))


def concat_net(seed=41, n=2, c=32, hw=18, branches=(24, 40, 16), oc=48, signed=False):
    """Branches of quantized convolutions joined by a Concat along the channels and consumed by another
    convolution, in the form the low-precision transformations leave (concat.cpp:42-190): every branch's
    FakeQuantize gets the same interval, the Concat takes the u8 (or i8) levels themselves and one per-tensor
    dequantization follows it.  Channel counts that are no multiples of 4 or 16 exercise every copy width.
    Returns (graph, feeds, meta)."""
    rng = np.random.default_rng(seed)
    x = rng.uniform(0, 1, (n, c, hw, hw)).astype(np.float32)
    net = QuantizedNet()
    g = net.g
    a0 = net.input("data", x.shape, 1.0)
    out_high = 3.0
    acts, params = [], []
    for i, oc_b in enumerate(branches):
        k = 3 if i % 2 else 1
        w = (rng.standard_normal((oc_b, c, k, k), dtype=np.float32) * np.float32(0.12 if k == 1 else 0.05)).astype(np.float32)
        b = (rng.standard_normal(oc_b, dtype=np.float32) * np.float32(0.3)).astype(np.float32)
        acts.append(net.conv(a0, w, b, out_high, pads=(k // 2, k // 2), signed=signed))
        params.append((w, b))
    assert all(a["scale"] == acts[0]["scale"] for a in acts)
    cat = dict(node=g.concat([a["node"] for a in acts], axis=1), scale=acts[0]["scale"])
    g.result(net.dequantize(cat), "cat")
    ct = sum(branches)
    w = (rng.standard_normal((oc, ct, 3, 3), dtype=np.float32) * np.float32(0.04)).astype(np.float32)
    b = (rng.standard_normal(oc, dtype=np.float32) * np.float32(0.2)).astype(np.float32)
    g.result(net.conv_f32(cat, w, b, pads=(1, 1), relu=True), "out")
    params.append((w, b))
    return g, dict(data=x), dict(concat=cat["node"], branches=[a["node"] for a in acts], params=params, out_high=out_high)


def per_channel_zero_point_net(seed=47, n=2, c=48, hw=17, oc=40, stride=1):
    """A depthwise convolution whose input is quantized per channel with asymmetric intervals: u8 levels with one
    integer zero point per channel in front of the GroupConvolution (the only place the transformations leave
    distinct per-channel zero points: convolution.cpp:97-120 broadcasts the Subtract constant over the channels,
    and only a grouped convolution's input may be quantized per channel), padded, so the halo must hold every
    channel's own level; then a dense 1 x 1 convolution to f32.  Returns (graph, feeds, meta)."""
    rng = np.random.default_rng(seed)
    x = rng.normal(0.3, 1.0, (n, c, hw, hw)).astype(np.float32)
    net = QuantizedNet()
    g = net.g
    lo = rng.uniform(-2.5, -0.5, c).astype(np.float32)
    hi = rng.uniform(0.8, 3.0, c).astype(np.float32)
    a0 = net.asymmetric_per_channel(g.parameter("data", x.shape), lo, hi)
    assert len(set(a0["zero_point"].tolist())) > 8
    w1 = (rng.standard_normal((c, 1, 3, 3), dtype=np.float32) * np.float32(0.3)).astype(np.float32)
    b1 = (rng.standard_normal(c, dtype=np.float32) * np.float32(0.2)).astype(np.float32)
    a1 = net.conv(a0, w1, b1, 2.5, strides=(stride, stride), pads=(1, 1), grouped=True)
    w2 = (rng.standard_normal((oc, c, 1, 1), dtype=np.float32) * np.float32(0.1)).astype(np.float32)
    b2 = (rng.standard_normal(oc, dtype=np.float32) * np.float32(0.2)).astype(np.float32)
    g.result(net.conv_f32(a1, w2, b2), "out")
    return g, dict(data=x), dict(acts=dict(a0=a0, a1=a1))


def matmul_zero_point_net(seed=53, batch=2, seq=48, hidden=128, ffn=192, r0=(-1.6, 2.9), r1=(-0.7, 1.9)):
    """Row-major (transformer) path with asymmetric u8 activations: LayerNorm -> FakeQuantize(u8, zero point) ->
    MatMul' -> Subtract(zero point x column sums of the weights) -> Add(bias over scale) -> FakeQuantize(u8, zero point; the
    dequantization folded into its range) -> MatMul' -> Subtract -> Add -> Multiply(s) -> + residual, i.e. what
    MatMulTransformation leaves when the activations in front of a MatMul have a zero point (mat_mul.cpp:95-121:
    the Subtract moves BEHIND the MatMul as zero point x weights).  Returns (graph, meta)."""
    rng = np.random.default_rng(seed)
    net = QuantizedNet()
    g = net.g
    nrm = lambda *shape, s=0.05: (rng.standard_normal(shape, dtype=np.float32) * np.float32(s)).astype(np.float32)
    x = g.parameter("hidden_states", (batch, seq, hidden))
    n = g.mvn(x, (-1,), True, 1e-5, True)
    h = g.add(g.multiply(n, g.constant(np.float32(1) + nrm(hidden))), g.constant(nrm(hidden) + np.float32(0.4)))

    def fq_u8(v, lo, hi, fold=None):
        d = lpt.decompose_fake_quantize(256, np.float32(lo), np.float32(hi), allow_zero_point=True)
        assert d["has_zero_point"] and d["precision"] == U8
        il, ih = (np.float32(lo), np.float32(hi)) if fold is None else lpt.fuse_elementwise(lpt.MULTIPLY, np.float32(lo), np.float32(hi), fold)
        q = g.fake_quantize(v, il, ih, d["new_low"], d["new_high"], 256, U8)
        return dict(node=q, scale=np.float32(d["scale"]).reshape(()), zero_point=np.float32(lpt.round_zero_point(d["shift"])).reshape(()))

    def linear(act, w, b):
        """MatMul' -> Subtract(zp * sum_k w) -> Add(b / s): returns (node, s[c])"""
        wq, s_w = lpt.quantize_weights(w, 255)
        s = (np.float32(act["scale"]) * s_w).astype(np.float32)
        params.append((w, b))
        y = g.matmul(act["node"], g.constant(wq, I8), False, True)
        # fold<MatMul>(broadcast(zero point) [1, K], weights): one f32 product per column, exact integers here
        corr = (np.full((1, wq.shape[1]), act["zero_point"], np.float32) @ wq.astype(np.float32).T).reshape(-1).astype(np.float32)
        y = g.subtract(y, g.constant(corr))
        return g.add(y, g.constant(lpt.swap_multiply_and_add(b, s))), s

    params = []
    a0 = fq_u8(h, r0[0], r0[1])
    y1, s1 = linear(a0, nrm(ffn, hidden), nrm(ffn, s=0.3))
    a1 = fq_u8(y1, r1[0], r1[1], fold=s1)
    y2, s2 = linear(a1, nrm(hidden, ffn), nrm(hidden, s=0.3))
    out = g.add(g.multiply(y2, g.constant(s2)), h)
    g.result(out, "out")
    return g, dict(norm=h, a0=a0["node"], a1=a1["node"], zero_points=(float(a0["zero_point"]), float(a1["zero_point"])),
                   linear=params)


def eltwise_net(seed=59, n=2, c=24, hw=14, oc=40):
    """Elementwise nodes that no convolution absorbs: two pooled, dequantized u8 branches added, ReLU and a
    FakeQuantize behind the Add (one kernel); the product of two f32 convolution results, clamped (one kernel, f32
    result); a FakeQuantize of that f32 value on its own; a Subtract with a per-channel constant on the left.
    Returns (graph, feeds, meta)."""
    rng = np.random.default_rng(seed)
    x = rng.uniform(0, 1, (n, c, hw, hw)).astype(np.float32)
    net = QuantizedNet()
    g = net.g
    a0 = net.input("data", x.shape, 1.0)
    w = lambda o, i, k, s: (rng.standard_normal((o, i, k, k), dtype=np.float32) * np.float32(s)).astype(np.float32)
    b = lambda o: (rng.standard_normal(o, dtype=np.float32) * np.float32(0.2)).astype(np.float32)
    a1 = net.conv(a0, w(oc, c, 3, 0.08), b(oc), 2.0, pads=(1, 1))
    a2 = net.conv(a0, w(oc, c, 1, 0.15), b(oc), 3.0)
    p1 = net.max_pool(a1, (3, 3), (1, 1), (1, 1))
    p2 = net.max_pool(a2, (3, 3), (1, 1), (1, 1))
    s = g.relu(g.add(net.dequantize(p1), net.dequantize(p2)))                 # Add of two dequantized byte tensors
    a3 = net.requantize(s, 4.0)
    f1 = net.conv_f32(a3, w(oc, oc, 1, 0.1), b(oc))
    f2 = net.conv_f32(a1, w(oc, oc, 3, 0.04), b(oc), pads=(1, 1))
    prod = g.clamp(g.multiply(f1, f2), -1.5, 2.5)                             # f32 x f32, Clamp behind it
    g.result(prod, "prod")
    a4 = net.requantize(prod, 2.5, signed=True)                               # FakeQuantize of a computed f32 value
    left = g.subtract(g.constant(net._channel(np.linspace(-1, 1, oc).astype(np.float32), 4)), net.dequantize(a4))
    g.result(left, "left")
    return g, dict(data=x), dict(acts=dict(a3=a3, a4=a4))
