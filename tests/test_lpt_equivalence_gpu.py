"""What the low-precision transformations promise, end to end: the transformed graph (integer weights, u8 / i8
activations, zero points as Subtracts, dequantization scales folded behind the convolution) computes the same function
as the graph it came from - FakeQuantize on the data and on the weights in front of a float convolution / MatMul -
up to f32 rounding.  The builders derive the transformed graph with the pinned steps of dldt_amd/lpt.py; here the
device result is compared with the ORIGINAL graph evaluated in float64 (the FakeQuantize levels taken from the oracle,
so both sides round the same inputs to the same levels).  A dropped or mis-signed term of the transformation - the zero
point times the weight sums, a scale on the wrong side of the bias, a group's scale on another group's channels -
moves the result by far more than the tolerance.

Layer parameters follow the reference's subgraph tests for quantized layers
(inference-engine/tests/functional/plugin/cpu/shared_tests_instances/subgraph_tests/quantized_group_convolution.cpp:
inputs [1,3,10,10] and [1,24,10,10], 3 groups, 3 / 24 / 48 output channels, 1x1 and 3x3 kernels, per-tensor and
per-channel quantization; quantized_mat_mul.cpp: u8 x i8 and i8 x i8 operands); the intervals are this file's own
(the reference draws them from its C++ generator) with zero points that are exact integers, so that rounding the
shift to a level (network_helper.cpp:485-494) changes nothing."""
import numpy as np
import pytest

from interp import evaluate

pytestmark = pytest.mark.gpu


def _fq_values(orc, x, lo, hi, levels=256):
    """FakeQuantize with output range = input range, as in the original graph (f32, reference arithmetic)"""
    shape = (1, -1, 1, 1) if np.ndim(lo) else ()
    lo, hi = np.asarray(lo, np.float32).reshape(shape), np.asarray(hi, np.float32).reshape(shape)
    return orc.fake_quantize(x, lo, hi, lo, hi, levels)


def _conv64(x, w, groups, bias, pad):
    import torch
    y = torch.nn.functional.conv2d(torch.from_numpy(x.astype(np.float64)), torch.from_numpy(w.astype(np.float64)),
                                   torch.from_numpy(bias.astype(np.float64)), padding=pad, groups=groups)
    return y.numpy()


# (per-channel intervals over 24 channels differ inside a group: the transformation leaves that layer in f32, and
# test_f32_layers_gpu.py::test_group_convolution_with_intervals_that_differ_inside_a_group runs those cells as such)
@pytest.mark.parametrize("c,oc,kernel,per_channel", [(c, oc, k, pc) for c in (3, 24) for oc in (3, 24, 48) for k in (1, 3)
                                                     for pc in (False, True) if not (pc and c != 3)])
def test_quantized_group_convolution_equals_its_float_graph(orc, c, oc, kernel, per_channel):
    from dldt_amd import builders, lpt
    G = 3
    rng = np.random.default_rng(c * 1000 + oc * 10 + kernel + 5 * per_channel)
    x = rng.normal(0.2, 1.2, (1, c, 10, 10)).astype(np.float32)
    w = (rng.standard_normal((oc, c // G, kernel, kernel)) * 0.3).astype(np.float32)
    b = (rng.standard_normal(oc) * 0.2).astype(np.float32)
    # intervals [-z / 64, (255 - z) / 64]: scale 1 / 64, zero point exactly z
    z = rng.integers(60, 200, c if per_channel else 1).astype(np.float32)
    z[z == 128] = 129            # [-128 / 64, 127 / 64] is the signed range itself: no zero point, i8 levels
    lo, hi = -z / np.float32(64), (np.float32(255) - z) / np.float32(64)
    net = builders.QuantizedNet()
    g = net.g
    p = g.parameter("data", x.shape)
    a = net.asymmetric_per_channel(p, lo, hi) if per_channel else net.asymmetric(p, lo[0], hi[0])
    np.testing.assert_array_equal(np.asarray(a["zero_point"]).reshape(-1), z)
    depthwise = c == G and oc == G
    pad = kernel // 2
    y = net.conv_f32(a, w, b, pads=(pad, pad), grouped=depthwise, groups=0 if depthwise else G)
    g.result(y, "out")
    want_graph, _ = evaluate(orc, g.nodes, {"data": x})
    req = g.compile().create_request()
    (got,) = req.infer(x)
    np.testing.assert_array_equal(got.view(np.uint32), want_graph["out"].view(np.uint32))     # the transformed graph, bit for bit
    # the original graph: FakeQuantize(data) and FakeQuantize(weights, 255 levels, +-max per output channel) in front
    # of a float GroupConvolution
    xq = _fq_values(orc, x, lo if per_channel else lo[0], hi if per_channel else hi[0])
    wq, s_w = lpt.quantize_weights(w, 255)
    w_fq = wq.astype(np.float64) * s_w.astype(np.float64).reshape(-1, 1, 1, 1)
    ref = _conv64(xq, w_fq, G, b, pad)
    assert np.abs(w_fq - w).max() <= np.abs(w).max() / 127                                      # the weights are on their grid
    np.testing.assert_allclose(got, ref, rtol=1e-4, atol=2e-5 * np.abs(ref).max())
    assert np.abs(ref).max() > 0.5


@pytest.mark.parametrize("lead", [(4,), (2, 3)])
@pytest.mark.parametrize("left,right", [("u8", "i8"), ("i8", "i8"), ("i8", "u8"), ("u8", "u8")])
def test_quantized_matmul_between_activations_equals_its_float_graph(orc, left, right, lead):
    """FakeQuantize(A) x FakeQuantize(B), both graph inputs, each to u8 levels of [0, hi] or to i8 symmetric (no zero
    point either way: MatMulTransformation rewrites no other MatMul between activations, mat_mul.cpp:231-236,
    :265-267, :290-292); after the transformation an integer MatMul and one Multiply by both scales"""
    from dldt_amd import lpt
    from dldt_amd.graph import Graph
    from dldt_amd.tensor import I8, U8
    rng = np.random.default_rng(11 + (left == "u8") + 2 * (right == "u8"))
    # (one or two batch dimensions; the graph inputs are rank 3 either way, the second form reshapes the quantized
    # tensors to rank 4 and walks the operands by an inner and an outer stride)
    nb = int(np.prod(lead))
    sa, sb = (nb, 64, 128), (nb, 128, 64)
    A = (rng.uniform(0, 1, sa) if left == "u8" else rng.normal(0, 0.4, sa)).astype(np.float32)
    B = (rng.uniform(0, 1.5, sb) if right == "u8" else rng.normal(0, 0.5, sb)).astype(np.float32)
    g = Graph()
    pa, pb = g.parameter("a", A.shape), g.parameter("b", B.shape)
    if left == "u8":
        lo_a, hi_a = np.float32(0), np.float32(1)
    else:
        hi_a = np.float32(1.0)
        lo_a = np.float32(-hi_a * np.float32(128) / np.float32(127))
    hi_b = np.float32(1.5)
    lo_b = np.float32(0) if right == "u8" else np.float32(-hi_b * np.float32(128) / np.float32(127))
    da, db = lpt.decompose_fake_quantize(256, lo_a, hi_a), lpt.decompose_fake_quantize(256, lo_b, hi_b)
    assert da["precision"] == (U8 if left == "u8" else I8) and db["precision"] == (U8 if right == "u8" else I8)
    assert not da.get("has_zero_point", False) and not db.get("has_zero_point", False)
    qa = g.fake_quantize(pa, lo_a, hi_a, da["new_low"], da["new_high"], 256, da["precision"])
    qb = g.fake_quantize(pb, lo_b, hi_b, db["new_low"], db["new_high"], 256, db["precision"])
    s = np.float32(da["scale"]) * np.float32(db["scale"])
    if len(lead) == 2:
        qa, qb = g.reshape(qa, lead + (64, 128)), g.reshape(qb, lead + (128, 64))
    g.result(g.multiply(g.matmul(qa, qb), g.constant(np.float32(s).reshape(()))), "out")
    want_graph, _ = evaluate(orc, g.nodes, {"a": A, "b": B})
    req = g.compile().create_request()
    (got,) = req.infer(A, B)
    np.testing.assert_array_equal(got.view(np.uint32), want_graph["out"].view(np.uint32))
    a_fq = orc.fake_quantize(A, lo_a, hi_a, lo_a, hi_a, 256).astype(np.float64)
    b_fq = orc.fake_quantize(B, lo_b, hi_b, lo_b, hi_b, 256).astype(np.float64)
    ref = (a_fq @ b_fq).reshape(got.shape)
    np.testing.assert_allclose(got, ref, rtol=1e-4, atol=2e-5 * np.abs(ref).max())
    assert np.abs(ref).max() > 1.0


def _fq64(v, hi):
    """FakeQuantize(0, hi) to 256 levels in float64: (levels, values)"""
    lv = np.rint(np.clip(v, 0.0, float(hi)) / float(hi) * 255.0)
    return lv, lv / 255.0 * float(hi)


def test_resnet_stack_follows_its_float_graph(orc):
    """A reduced ResNet (stem, max-pool, two stages of bottleneck blocks with projection and identity shortcuts, global
    average pool, FC) as the builder derives its transformed graph, against the graph it stands for: FakeQuantize
    behind every ReLU, on the pooled features and on the weights, everything else in float64.  The two differ only
    where f32 rounding puts a value on the other side of a level boundary, and such a flip moves later values by a
    fraction of a level: at this size every activation keeps its level (one level off is allowed for), the logits agree to
    a fraction of a percent of their range.  (A wrong bias or residual scale, a dropped dequantization or a
    misplaced Multiply shows as whole levels everywhere.)"""
    import torch
    import torch.nn.functional as F
    from dldt_amd import builders, lpt
    stages = [(16, 2, 1), (32, 2, 2)]
    g, meta = builders.resnet50(batch=2, res=32, width=16, classes=10, seed=7, stages=stages)
    P, R, acts = meta["params"], meta["ranges"], meta["acts"]
    x = np.random.default_rng(3).uniform(0, 1, (2, 3, 32, 32)).astype(np.float32)
    req = g.compile().create_request()
    (logits,) = req.infer(x)

    def conv(name, v, stride=1, pad=0):
        wq, s_w = lpt.quantize_weights(P[name + ".w"], 255)
        w = wq.astype(np.float64) * s_w.astype(np.float64).reshape((-1,) + (1,) * (wq.ndim - 1))
        return F.conv2d(v, torch.from_numpy(w), torch.from_numpy(P[name + ".b"].astype(np.float64)), stride=stride, padding=pad)

    worst = {}

    def check(name, levels64):
        dev = req.tensor(acts[name]["node"], fused_ok=True)
        if dev is None:             # kept in LDS between two convolutions that run as one kernel: the next tensor tells
            return
        dev = dev.astype(np.int64)
        d = np.abs(dev - levels64.astype(np.int64))
        worst[name] = (float((d > 0).mean()), int(d.max()))
        assert d.max() <= 1 and (d > 0).mean() < 0.002, (name, worst[name])

    lv, v = _fq64(x.astype(np.float64), R["input"])
    np.testing.assert_array_equal(req.tensor(acts["input"]["node"]), orc.fake_quantize(x, np.float32(0), np.float32(R["input"]),
                                                                                      np.float32(0), np.float32(255), 256))
    v = torch.from_numpy(v)
    lv, v = _fq64(conv("conv1", v, 2, 3).numpy(), R["conv1"])
    check("conv1", lv)
    v = F.max_pool2d(torch.from_numpy(v), 3, 2, 1)
    for si, (_, blocks, stride) in enumerate(stages):
        for bi in range(blocks):
            p = "layer%d.%d" % (si + 1, bi)
            s = stride if bi == 0 else 1
            lv, ya = _fq64(conv(p + ".a", v).numpy(), R[p + ".a"])
            check(p + ".a", lv)
            lv, yb = _fq64(conv(p + ".b", torch.from_numpy(ya), s, 1).numpy(), R[p + ".b"])
            check(p + ".b", lv)
            yc = conv(p + ".c", torch.from_numpy(yb))
            sc = conv(p + ".ds", v, s) if bi == 0 else v
            lv, out = _fq64((yc + sc).numpy(), R[p + ".out"])
            check(p + ".out", lv)
            v = torch.from_numpy(out)
    lv, pooled = _fq64(v.mean(dim=(2, 3)).numpy(), R["pool"])
    check("pool", lv.reshape(req.tensor(acts["pool"]["node"]).shape))
    wq, s_w = lpt.quantize_weights(P["fc.w"], 255)
    ref = pooled @ (wq.astype(np.float64) * s_w.astype(np.float64).reshape(-1, 1)).T + P["fc.b"].astype(np.float64)
    span = ref.max() - ref.min()
    assert np.abs(logits - ref).max() < 0.01 * span, (np.abs(logits - ref).max(), span, worst)
    assert np.array_equal(np.argmax(logits, 1), np.argmax(ref, 1))
    print(worst)


def test_mobilenet_stack_follows_its_float_graph(orc):
    """The same for a reduced MobileNetV2: ReLU6 layers quantized to u8 levels of [0, max], depthwise layers, linear
    bottlenecks quantized to symmetric i8, the residual Add of a block's input (an i8 value, dequantized) in front
    of the next FakeQuantize, global average pool and FC."""
    import torch
    import torch.nn.functional as F
    from dldt_amd import builders, lpt
    blocks = [(1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 2, 1)]
    g, meta = builders.mobilenet_v2(batch=2, res=32, width=1.0, classes=10, seed=9, blocks=blocks, last=64)
    P, R, acts = meta["params"], meta["ranges"], meta["acts"]
    x = np.random.default_rng(4).uniform(0, 1, (2, 3, 32, 32)).astype(np.float32)
    req = g.compile().create_request()
    (logits,) = req.infer(x)

    def conv(name, v, stride=1, pad=0, groups=1):
        wq, s_w = lpt.quantize_weights(P[name + ".w"], 255)
        w = wq.astype(np.float64) * s_w.astype(np.float64).reshape(-1, 1, 1, 1)
        return F.conv2d(v, torch.from_numpy(w), torch.from_numpy(P[name + ".b"].astype(np.float64)), stride=stride,
                        padding=pad, groups=groups)

    def fq_signed(v, m):
        hi = float(m)
        lo = -hi * 128.0 / 127.0
        lv = np.rint((np.clip(v, lo, hi) - lo) / (hi - lo) * 255.0)
        return lv - 128, lo + lv / 255.0 * (hi - lo)

    worst = {}

    def check(name, levels64):
        dev = req.tensor(acts[name]["node"], fused_ok=True)
        if dev is None:             # kept in LDS between two convolutions that run as one kernel: the next tensor tells
            return
        dev = dev.astype(np.int64)
        d = np.abs(dev - levels64.astype(np.int64))
        worst[name] = (float((d > 0).mean()), int(d.max()))
        assert d.max() <= 1 and (d > 0).mean() < 0.002, (name, worst[name])

    _, v = _fq64(x.astype(np.float64), R["input"])
    v = torch.from_numpy(v)
    names = {n for n, *_ in builders._mbv2_layers(1.0, blocks, 64)}
    block_in = None
    linear = 0
    for name, kind, ic, oc, stride, residual in builders._mbv2_layers(1.0, blocks, 64):
        if name.endswith(".expand") or (kind == "dw" and name[:-3] + ".expand" not in names):
            block_in = v
        if kind in ("conv3", "pw_relu6", "dw"):
            y = conv(name, v, stride, 1 if kind != "pw_relu6" else 0, ic if kind == "dw" else 1)
            lv, out = _fq64(np.clip(y.numpy(), 0.0, 6.0), R[name])
        else:
            y = conv(name, v)
            if residual:
                y = y + block_in
            lv, out = fq_signed(y.numpy(), R[name])
            linear += 1
        check(name, lv)
        v = torch.from_numpy(out)
    assert linear == 5 and any(r for *_, r in builders._mbv2_layers(1.0, blocks, 64))
    lv, pooled = _fq64(v.mean(dim=(2, 3)).numpy(), R["pool"])
    check("pool", lv.reshape(req.tensor(acts["pool"]["node"]).shape))
    wq, s_w = lpt.quantize_weights(P["fc.w"], 255)
    ref = pooled @ (wq.astype(np.float64) * s_w.astype(np.float64).reshape(-1, 1)).T + P["fc.b"].astype(np.float64)
    span = ref.max() - ref.min()
    assert np.abs(logits - ref).max() < 0.01 * span, (np.abs(logits - ref).max(), span, worst)
    print(worst)


@pytest.mark.parametrize("unsigned_probs", [False, True])
def test_encoder_layer_follows_its_float_graph(orc, monkeypatch, unsigned_probs):
    """One encoder layer (attention with i8 or u8 probabilities, residual Adds, LayerNorms, Gelu, six MatMuls against
    quantized weights) against its float64 original with a FakeQuantize wherever the transformed graph holds a byte
    tensor.  Softmax, LayerNorm and Gelu are f32 approximations on the device, so a few values land on the other
    side of a level boundary: at most one level off, in under one percent of any tensor."""
    from scipy.special import erf
    from dldt_amd import builders, lpt
    hidden, heads, ffn, batch, seq = 128, 2, 256, 2, 64
    D = hidden // heads
    r = dict(builders.BERT_RANGES)
    r.update(q=0.12, k=0.9, v=0.9, ctx=0.6)
    g, meta = builders.bert_encoder(layers=1, hidden=hidden, heads=heads, ffn=ffn, batch=batch, seq=seq, seed=7,
                                    ranges=dict(q=0.12, k=0.9, v=0.9, ctx=0.6), unsigned_probs=unsigned_probs)
    x = np.random.default_rng(70).normal(0, 1, (batch, seq, hidden)).astype(np.float32)
    monkeypatch.setenv("HIPIE_KEEP_F32", "1")
    monkeypatch.setenv("HIPIE_FUSE_ATTENTION", "0")        # the quantized probabilities are a tensor to look at
    req = g.compile().create_request()
    (y,) = req.infer(x)
    monkeypatch.setenv("HIPIE_FUSE_ATTENTION", "1")
    (y_fused,) = g.compile().create_request().infer(x)
    np.testing.assert_array_equal(y_fused.view(np.uint32), y.view(np.uint32))
    L = meta["layers"][0]

    def fq_s(v, m):
        hi = float(m)
        lo = -hi * 128.0 / 127.0
        lv = np.rint((np.clip(v, lo, hi) - lo) / (hi - lo) * 255.0)
        return lv - 128, lo + lv / 255.0 * (hi - lo)

    def linear(i, v):
        w, b = meta["linear"][i]
        wq, s_w = lpt.quantize_weights(w, 255)
        return v @ (wq.astype(np.float64) * s_w.astype(np.float64).reshape(-1, 1)).T + b.astype(np.float64)

    def norm(i, v):
        gamma, beta = meta["norm"][i]
        m = v.mean(-1, keepdims=True)
        var = ((v - m) ** 2).mean(-1, keepdims=True)
        return (v - m) / np.sqrt(var + 1e-5) * gamma.astype(np.float64) + beta.astype(np.float64)

    def heads_of(v):
        return v.reshape(batch, seq, heads, D).transpose(0, 2, 1, 3)

    worst = {}

    def check(name, levels64):
        dev = req.matrix(L[name]).astype(np.int64).reshape(levels64.shape)
        d = np.abs(dev - levels64.astype(np.int64))
        worst[name] = (float((d > 0).mean()), int(d.max()))
        assert d.max() <= 1 and (d > 0).mean() < 0.01, (name, worst[name])

    x64 = x.astype(np.float64)
    lv, xq = fq_s(x64, r["x"]); check("xq", lv)
    lv, q = fq_s(linear(0, xq), r["q"]); check("q", lv)
    lv, k = fq_s(linear(1, xq), r["k"]); check("k", lv)
    lv, v = fq_s(linear(2, xq), r["v"]); check("v", lv)
    s = heads_of(q) @ heads_of(k).transpose(0, 1, 3, 2)
    e = np.exp(s - s.max(-1, keepdims=True))
    p = e / e.sum(-1, keepdims=True)
    if unsigned_probs:
        lv, pq = _fq64(p, r["p"])
    else:
        lv, pq = fq_s(p, r["p"])
    check("pq", lv)
    ctx = (pq @ heads_of(v)).transpose(0, 2, 1, 3).reshape(batch, seq, hidden)
    lv, cq = fq_s(ctx, r["ctx"]); check("ctxq", lv)
    h1 = norm(0, linear(3, cq) + x64)
    lv, h1q = fq_s(h1, r["h1"]); check("h1q", lv)
    f = linear(4, h1q)
    gl = 0.5 * f * (1.0 + erf(f / np.sqrt(2.0)))
    lv, gq = fq_s(gl, r["g"]); check("gq", lv)
    ref = norm(1, linear(5, gq) + h1)
    np.testing.assert_allclose(y, ref, rtol=0, atol=0.02 * np.abs(ref).max())
    assert np.abs(y - ref).mean() < 1e-3 * np.abs(ref).max()
    print(worst)


def test_weight_matmuls_with_zero_points_equal_their_float_graph(orc):
    """MatMuls against quantized weights whose activations are u8 levels with a zero point: the transformation moves the
    zero point BEHIND the MatMul (zero point x column sums of the weights, mat_mul.cpp:95-121).  Intervals with exact
    integer zero points (90 at scale 1/64, 45 at scale 1/128), so the transformed graph is the original one up to
    f32 rounding.  The original starts from the device's LayerNorm output (an f32 approximation on the device)."""
    from dldt_amd import builders, lpt
    r0 = (-90 / 64, 165 / 64)
    r1 = (-45 / 128, 210 / 128)
    g, meta = builders.matmul_zero_point_net(r0=r0, r1=r1)
    assert meta["zero_points"] == (90.0, 45.0)
    x = np.random.default_rng(5).normal(0, 1, (2, 48, 128)).astype(np.float32)
    req = g.compile().create_request()
    (out,) = req.infer(x)
    h = req.matrix(meta["norm"]).astype(np.float64).reshape(2, 48, 128)

    def fq(v, r):
        lo, hi = float(np.float32(r[0])), float(np.float32(r[1]))
        lv = np.rint((np.clip(v, lo, hi) - lo) / (hi - lo) * 255.0)
        return lv, lo + lv / 255.0 * (hi - lo)

    def linear(i, v):
        w, b = meta["linear"][i]
        wq, s_w = lpt.quantize_weights(w, 255)
        return v @ (wq.astype(np.float64) * s_w.astype(np.float64).reshape(-1, 1)).T + b.astype(np.float64)

    lv0, a0 = fq(h, r0)
    d = np.abs(req.matrix(meta["a0"]).astype(np.int64).reshape(lv0.shape) - lv0.astype(np.int64))
    assert d.max() <= 1 and (d > 0).mean() < 0.002
    lv1, a1 = fq(linear(0, a0), r1)
    d = np.abs(req.matrix(meta["a1"]).astype(np.int64).reshape(lv1.shape) - lv1.astype(np.int64))
    assert d.max() <= 1 and (d > 0).mean() < 0.002
    assert lv0.min() == 0 and lv0.max() == 255 and len(np.unique(lv1)) > 200       # both intervals are used to their ends
    ref = linear(1, a1) + h
    np.testing.assert_allclose(out, ref, rtol=0, atol=0.01 * np.abs(ref).max())
    assert np.abs(out - ref).mean() < 2e-4 * np.abs(ref).max()


@pytest.mark.parametrize("signed", [False, True])
def test_concat_of_quantized_branches_equals_its_float_graph(orc, signed):
    """three convolution branches, each behind the same FakeQuantize interval, concatenated and convolved again:
    the transformed graph concatenates the levels and dequantizes once (concat.cpp:42-190)"""
    import torch
    import torch.nn.functional as F
    from dldt_amd import builders, lpt
    g, feeds, meta = builders.concat_net(signed=signed)
    req = g.compile().create_request()
    cat_dev, out_dev = req.infer(feeds["data"])

    def conv(i, v):
        w, b = meta["params"][i]
        wq, s_w = lpt.quantize_weights(w, 255)
        return F.conv2d(v, torch.from_numpy(wq.astype(np.float64) * s_w.astype(np.float64).reshape(-1, 1, 1, 1)),
                        torch.from_numpy(b.astype(np.float64)), padding=w.shape[-1] // 2)

    _, x = _fq64(feeds["data"].astype(np.float64), 1.0)
    x = torch.from_numpy(x)
    hi = float(meta["out_high"])
    lo = -hi * 128.0 / 127.0 if signed else 0.0
    parts = []
    for i in range(len(meta["branches"])):
        v = conv(i, x).numpy()
        lv = np.rint((np.clip(v, lo, hi) - lo) / (hi - lo) * 255.0)
        parts.append(lo + lv / 255.0 * (hi - lo))
    cat = np.concatenate(parts, axis=1)
    np.testing.assert_allclose(cat_dev, cat, rtol=0, atol=1.01 * (hi - lo) / 255.0)       # at most one level anywhere
    assert (np.abs(cat_dev - cat) > 1e-5).mean() < 0.002
    ref = np.maximum(conv(len(parts), torch.from_numpy(cat)).numpy(), 0.0)
    np.testing.assert_allclose(out_dev, ref, rtol=0, atol=0.01 * ref.max())
    assert np.abs(out_dev - ref).mean() < 2e-4 * ref.max()
