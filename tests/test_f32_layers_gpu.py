"""Layers the low-precision transformations leave in f32 - no FakeQuantize in front of them, or intervals the
transformation does not take (convolution.cpp:84-120, weightable_layer_transformation.cpp: per-channel intervals that
differ inside a group) - run as the graph says: reference::convolution<float> / group_convolution<float> / matmul<float>
and fake_quantize<float>, every sum in the reference's order.  The device result is compared with the oracle's
evaluation of the same graph bit for bit (f32 words as uint32), and where the test states a float64 original, with
that as well."""
import numpy as np
import pytest

from interp import evaluate

pytestmark = pytest.mark.gpu


def _bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def _folded_weights(orc, w, levels=255):
    """FakeQuantize(weights, +-max per output channel) as constant folding leaves it: an f32 constant"""
    m = np.abs(w).reshape(w.shape[0], -1).max(1).astype(np.float32).reshape((-1,) + (1,) * (w.ndim - 1))
    return orc.fake_quantize(w, -m, m, -m, m, levels)


@pytest.mark.parametrize("kernel", [1, 3])
@pytest.mark.parametrize("oc", [3, 24, 48])
def test_group_convolution_with_intervals_that_differ_inside_a_group(orc, oc, kernel):
    """the cells of quantized_group_convolution.cpp that the transformation leaves alone: 24 channels in 3 groups, one
    FakeQuantize interval per CHANNEL; FakeQuantize keeps its f32 result and the GroupConvolution its f32 weights"""
    import torch
    from dldt_amd.graph import Graph
    G, c = 3, 24
    rng = np.random.default_rng(oc * 10 + kernel)
    x = rng.normal(0.2, 1.2, (1, c, 10, 10)).astype(np.float32)
    w = (rng.standard_normal((oc, c // G, kernel, kernel)) * 0.3).astype(np.float32)
    b = (rng.standard_normal(oc) * 0.2).astype(np.float32)
    z = rng.integers(60, 200, c).astype(np.float32)
    lo, hi = (-z / np.float32(64)).reshape(1, c, 1, 1), ((np.float32(255) - z) / np.float32(64)).reshape(1, c, 1, 1)
    w_fq = _folded_weights(orc, w)
    g = Graph()
    p = g.parameter("data", x.shape)
    q = g.fake_quantize(p, lo, hi, lo, hi, 256)
    pad = kernel // 2
    y = g.convolution(q, g.constant(w_fq.reshape(G, oc // G, c // G, kernel, kernel)), pads_begin=(pad, pad), pads_end=(pad, pad), grouped=True)
    g.result(g.add(y, g.constant(b.reshape(1, oc, 1, 1))), "out")
    want, _ = evaluate(orc, g.nodes, {"data": x})
    plan = g.compile()
    (got,) = plan.create_request().infer(x)
    np.testing.assert_array_equal(_bits(got), _bits(want["out"]))
    kinds = {plan.steps[i]["type"]: plan.step_rt_info(i, "runtimePrecision") for i in range(len(plan.steps))}
    assert kinds["GroupConvolution"] == "FP32" and kinds["FakeQuantize"] == "FP32"
    xq = orc.fake_quantize(x, lo, hi, lo, hi, 256).astype(np.float64)
    ref = torch.nn.functional.conv2d(torch.from_numpy(xq), torch.from_numpy(w_fq.astype(np.float64)), torch.from_numpy(b.astype(np.float64)),
                                     padding=pad, groups=G).numpy()
    np.testing.assert_allclose(got, ref, rtol=1e-4, atol=2e-5 * np.abs(ref).max())
    assert np.abs(ref).max() > 0.5


@pytest.mark.parametrize("case", [
    dict(c=3, oc=16, k=(3, 3), s=(2, 2), d=(1, 1), pb=(1, 1), pe=(1, 1), hw=(17, 13), groups=1),
    dict(c=8, oc=12, k=(3, 2), s=(1, 2), d=(2, 1), pb=(2, 0), pe=(1, 1), hw=(9, 11), groups=1),
    dict(c=12, oc=8, k=(1, 1), s=(1, 1), d=(1, 1), pb=(0, 0), pe=(0, 0), hw=(5, 7), groups=4),
    dict(c=6, oc=6, k=(3, 3), s=(1, 1), d=(1, 1), pb=(1, 1), pe=(1, 1), hw=(8, 8), groups=6),
    dict(c=5, oc=7, k=(5, 5), s=(3, 3), d=(1, 1), pb=(2, 2), pe=(2, 2), hw=(16, 16), groups=1),
])
def test_f32_convolution_of_a_graph_input(orc, case):
    """an unquantized first layer: the f32 graph input (NCHW, as the request holds it) straight into the convolution;
    strides, dilations, uneven pads, groups; the oracle's float convolution is pinned against the reference's own
    vectors and the compiled reference headers in test_oracle.py"""
    from dldt_amd.graph import Graph
    rng = np.random.default_rng(case["c"] * 100 + case["oc"])
    G = case["groups"]
    x = rng.normal(0, 1, (2, case["c"]) + case["hw"]).astype(np.float32)
    w = rng.normal(0, 0.4, (case["oc"], case["c"] // G) + case["k"]).astype(np.float32)
    g = Graph()
    p = g.parameter("data", x.shape)
    wc = g.constant(w.reshape((G, case["oc"] // G, case["c"] // G) + case["k"]) if G > 1 else w)
    y = g.convolution(p, wc, strides=case["s"], dilations=case["d"], pads_begin=case["pb"], pads_end=case["pe"], grouped=G > 1)
    g.result(y, "out")
    want, _ = evaluate(orc, g.nodes, {"data": x})
    (got,) = g.compile().create_request().infer(x)
    assert got.shape == want["out"].shape
    np.testing.assert_array_equal(_bits(got), _bits(want["out"]))


def test_f32_first_layer_in_front_of_quantized_layers(orc):
    """f32 stem (Convolution, bias, ReLU) -> FakeQuantize to u8 levels -> quantized 3 x 3 convolution: the f32 island
    hands an NHWC f32 tensor to the elementwise step that quantizes it, and the integer kernels take over"""
    from dldt_amd import builders
    rng = np.random.default_rng(91)
    x = rng.uniform(0, 1, (2, 3, 20, 20)).astype(np.float32)
    w0 = rng.normal(0, 0.3, (16, 3, 3, 3)).astype(np.float32)
    b0 = rng.normal(0, 0.1, 16).astype(np.float32)
    w1 = rng.normal(0, 0.1, (32, 16, 3, 3)).astype(np.float32)
    b1 = rng.normal(0, 0.1, 32).astype(np.float32)
    net = builders.QuantizedNet()
    g = net.g
    p = g.parameter("data", x.shape)
    y = g.relu(g.add(g.convolution(p, g.constant(w0), strides=(2, 2), pads_begin=(1, 1), pads_end=(1, 1)), g.constant(b0.reshape(1, 16, 1, 1))))
    a = net.requantize(y, 2.0)
    out = net.conv_f32(a, w1, b1, pads=(1, 1), relu=True)
    g.result(out, "out")
    want, kept = evaluate(orc, g.nodes, {"data": x}, keep=[a["node"]])
    plan = g.compile()
    req = plan.create_request()
    (got,) = req.infer(x)
    np.testing.assert_array_equal(req.tensor(a["node"]), kept[a["node"]])
    np.testing.assert_array_equal(_bits(got), _bits(want["out"]))
    types = [plan.steps[i]["type"] for i in range(len(plan.steps))]
    assert types[0] == "Convolution" and plan.step_rt_info(0, "runtimePrecision") == "FP32"
    assert plan.step_rt_info(types.index("Convolution", 1), "runtimePrecision") == "U8"


@pytest.mark.parametrize("transposed", [False, True])
def test_f32_fully_connected_tail_behind_quantized_features(orc, transposed):
    """quantized features [N, C, 1, 1] -> Convert, Multiply (their dequantization) -> Reshape -> MatMul with f32 weights
    -> Add(bias): the kernel reads the level bytes and dequantizes them as the three nodes say"""
    from dldt_amd import builders
    from dldt_amd.tensor import F32
    rng = np.random.default_rng(92 + transposed)
    N, C, OC = 5, 70, 19
    x = rng.uniform(0, 3, (N, C, 1, 1)).astype(np.float32)
    w = rng.normal(0, 0.2, (OC, C) if transposed else (C, OC)).astype(np.float32)
    b = rng.normal(0, 0.1, OC).astype(np.float32)
    net = builders.QuantizedNet()
    g = net.g
    a = net.input("data", x.shape, 2.55)
    f = g.reshape(net.dequantize(a), (N, C))
    y = g.add(g.matmul(f, g.constant(w), False, transposed), g.constant(b.reshape(1, OC)))
    g.result(y, "logits")
    want, _ = evaluate(orc, g.nodes, {"data": x})
    (got,) = g.compile().create_request().infer(x)
    assert got.shape == (N, OC)
    np.testing.assert_array_equal(_bits(got), _bits(want["logits"]))


def test_f32_fake_quantize_between_layers(orc):
    """quantized convolution with an f32 result -> FakeQuantize that keeps f32 (per-channel intervals, output range other
    than the input range, 16 levels) -> f32 convolution"""
    from dldt_amd import builders
    rng = np.random.default_rng(93)
    x = rng.uniform(0, 2.55, (1, 8, 12, 12)).astype(np.float32)
    w0 = rng.normal(0, 0.2, (10, 8, 3, 3)).astype(np.float32)
    b0 = rng.normal(0, 0.1, 10).astype(np.float32)
    w1 = rng.normal(0, 0.3, (4, 10, 1, 1)).astype(np.float32)
    net = builders.QuantizedNet()
    g = net.g
    a = net.input("data", x.shape, 2.55)
    y = net.conv_f32(a, w0, b0, pads=(1, 1))
    il = rng.uniform(-1.5, -0.5, (1, 10, 1, 1)).astype(np.float32)
    ih = rng.uniform(0.5, 1.5, (1, 10, 1, 1)).astype(np.float32)
    q = g.fake_quantize(y, il, ih, np.float32(-1), np.float32(3), 16)
    g.result(g.convolution(q, g.constant(w1)), "out")
    want, kept = evaluate(orc, g.nodes, {"data": x}, keep=[q])
    req = g.compile().create_request()
    (got,) = req.infer(x)
    np.testing.assert_array_equal(_bits(req.tensor(q)), _bits(kept[q]))
    assert len(np.unique(kept[q])) == 16
    np.testing.assert_array_equal(_bits(got), _bits(want["out"]))


def test_mean_and_scale_in_front_of_the_first_fake_quantize(orc):
    """Parameter -> Subtract(mean[c]) -> Multiply(scale[c]) -> FakeQuantize(u8) -> quantized convolution: the
    preprocessing nodes a converted model keeps on its input read the request's NCHW buffer through an NHWC copy"""
    from dldt_amd import builders
    rng = np.random.default_rng(94)
    x = rng.uniform(0, 255, (2, 3, 16, 16)).astype(np.float32)
    mean = np.array([123.675, 116.28, 103.53], np.float32).reshape(1, 3, 1, 1)
    scale = (np.float32(1) / np.array([58.395, 57.12, 57.375], np.float32)).reshape(1, 3, 1, 1)
    w = rng.normal(0, 0.2, (8, 3, 3, 3)).astype(np.float32)
    b = rng.normal(0, 0.1, 8).astype(np.float32)
    net = builders.QuantizedNet()
    g = net.g
    p = g.parameter("data", x.shape)
    y = g.multiply(g.subtract(p, g.constant(mean)), g.constant(scale))
    a = net.asymmetric(y, -120 / 64, 135 / 64)     # scale 1 / 64, zero point 120 exactly
    assert a["zero_point"] == 120
    g.result(net.conv_f32(a, w, b, pads=(1, 1)), "out")
    want, kept = evaluate(orc, g.nodes, {"data": x}, keep=[a["node"]])
    plan = g.compile()
    req = plan.create_request()
    (got,) = req.infer(x)
    np.testing.assert_array_equal(req.tensor(a["node"]), kept[a["node"]])
    np.testing.assert_array_equal(_bits(got), _bits(want["out"]))
    assert [plan.steps[i]["type"] for i in range(len(plan.steps))][0] == "Reorder"


def test_f32_branches_pool_and_concat(orc):
    """an unquantized stem with two branches: f32 convolution -> ReLU -> MaxPool (f32), a second f32 convolution of the
    input with stride 2, Concat of both along the channels (f32), FakeQuantize to u8 levels, quantized convolution"""
    from dldt_amd import builders
    rng = np.random.default_rng(95)
    x = rng.uniform(-1, 1, (2, 3, 18, 18)).astype(np.float32)
    w0 = rng.normal(0, 0.3, (10, 3, 3, 3)).astype(np.float32)
    w1 = rng.normal(0, 0.3, (6, 3, 1, 1)).astype(np.float32)
    w2 = rng.normal(0, 0.1, (8, 16, 1, 1)).astype(np.float32)
    b2 = rng.normal(0, 0.1, 8).astype(np.float32)
    net = builders.QuantizedNet()
    g = net.g
    p = g.parameter("data", x.shape)
    a = g.max_pool(g.relu(g.convolution(p, g.constant(w0), pads_begin=(1, 1), pads_end=(1, 1))), (3, 3), (2, 2), (1, 1), (1, 1))
    b = g.convolution(p, g.constant(w1), strides=(2, 2))
    cat = g.concat([a, b], axis=1)
    q = net.requantize(g.relu(cat), 1.5)
    g.result(net.conv_f32(q, w2, b2), "out")
    want, kept = evaluate(orc, g.nodes, {"data": x}, keep=[cat, q["node"]])
    plan = g.compile()
    req = plan.create_request()
    (got,) = req.infer(x)
    np.testing.assert_array_equal(_bits(req.tensor(cat)), _bits(kept[cat]))
    np.testing.assert_array_equal(req.tensor(q["node"]), kept[q["node"]])
    np.testing.assert_array_equal(_bits(got), _bits(want["out"]))
    assert all(g.query())


@pytest.mark.parametrize("classes", [1000, 1001, 10])
def test_classifier_softmax(orc, classes):
    """... -> global average pool -> FC -> Softmax over the classes ([N, C], axis 1 or -1): the tail public
    classification models end with.  The logits in front of it bit for bit; the probabilities to rounding (exp is the
    device's), every row summing to one"""
    from dldt_amd import builders
    rng = np.random.default_rng(classes)
    x = rng.uniform(0, 1, (5, 16, 12, 12)).astype(np.float32)
    net = builders.QuantizedNet()
    g = net.g
    a0 = net.input("data", x.shape, 1.0)
    a1 = net.conv(a0, (rng.standard_normal((64, 16, 3, 3)) * 0.08).astype(np.float32), np.zeros(64, np.float32), 2.0, pads=(1, 1))
    pooled = g.avg_pool(net.dequantize(a1), (12, 12), (1, 1), (0, 0), (0, 0))
    q = net.requantize(pooled, 1.0)
    flat = dict(node=g.reshape(q["node"], (5, 64)), scale=q["scale"])
    logits = net.conv_f32(flat, (rng.standard_normal((classes, 64)) * 0.5).astype(np.float32), (rng.standard_normal(classes)).astype(np.float32),
                          matmul=True)
    g.result(logits, "logits")
    prob = g.softmax(logits, axis=-1 if classes == 10 else 1)
    g.result(prob, "prob")
    want, _ = evaluate(orc, g.nodes, {"data": x})
    plan = g.compile()
    assert [s["type"] for s in plan.steps].count("Softmax") == 1
    idx = [s["type"] for s in plan.steps].index("Softmax")
    assert plan.step_rt_info(idx, "runtimePrecision") == "FP32"
    req = plan.create_request()
    got = dict(zip([o["name"] for o in plan.outputs], req.infer(x)))
    np.testing.assert_array_equal(_bits(got["logits"]), _bits(want["logits"]))
    assert got["prob"].shape == (5, classes) and np.ptp(want["logits"]) > 4
    np.testing.assert_allclose(got["prob"], want["prob"], rtol=3e-6, atol=1e-9)
    np.testing.assert_allclose(got["prob"].sum(1), 1.0, rtol=1e-6)
    assert all(g.query())


def test_softmax_over_the_channels_of_a_feature_map(orc):
    """a segmentation or detection head: Softmax along axis 1 of [N, C, H, W] (21 classes per pixel), on an f32
    convolution's result and on the dequantized levels of a quantized one"""
    from dldt_amd import builders
    rng = np.random.default_rng(2121)
    x = rng.uniform(0, 1, (2, 8, 9, 11)).astype(np.float32)
    net = builders.QuantizedNet()
    g = net.g
    a0 = net.input("data", x.shape, 1.0)
    head = net.conv_f32(a0, (rng.standard_normal((21, 8, 3, 3)) * 0.6).astype(np.float32), rng.standard_normal(21).astype(np.float32), pads=(1, 1))
    g.result(g.softmax(head, axis=1), "per_pixel")
    a1 = net.conv(a0, (rng.standard_normal((21, 8, 1, 1)) * 0.5).astype(np.float32), np.zeros(21, np.float32), 3.0, signed=True)
    g.result(g.softmax(net.dequantize(a1), axis=-3), "of_levels")
    want, _ = evaluate(orc, g.nodes, {"data": x})
    plan = g.compile()
    assert [s["type"] for s in plan.steps].count("Softmax") == 2
    req = plan.create_request()
    got = dict(zip([o["name"] for o in plan.outputs], req.infer(x)))
    for name in ("per_pixel", "of_levels"):
        assert got[name].shape == (2, 21, 9, 11)
        np.testing.assert_allclose(got[name], want[name], rtol=3e-6, atol=1e-9, err_msg=name)
        np.testing.assert_allclose(got[name].sum(1), 1.0, rtol=1e-6)
    assert want["per_pixel"].max() > 0.5
    assert all(g.query())
