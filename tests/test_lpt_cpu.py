"""The restated LPT load-time arithmetic (include/hipie.h section 3) against the constants the
reference's own LPT unit tests expect (tests/golden/lpt.json), and the planner's fusion decisions in
a dry run without a device."""
import json
import os

import numpy as np
import pytest

from dldt_amd import lpt

G = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "lpt.json")))
PREC = {"u8": 40, "i8": 50, None: None}


@pytest.mark.parametrize("case", G["precision_details"]["cases"])
def test_precision_details(case):
    prec, neg, zp = lpt.precision_details(case["levels"], np.float32(case["out_low"]), np.float32(case["out_high"]))
    assert prec == PREC[case["precision"]] and neg == case["has_negative"] and zp == case["has_zero_point"]


@pytest.mark.parametrize("case", G["decompose"]["cases"])
def test_decompose_scale_shift(case):
    import ctypes
    from dldt_amd._lib import check, lib
    ol, oh = np.array([case["out_low"]], np.float32), np.array([case["out_high"]], np.float32)
    sc, sh, nl, nh = (np.empty(1, np.float32) for _ in range(4))
    p = lambda a: a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))  # noqa: E731
    check(lib().hipie_lpt_decompose_fake_quantize(p(ol), p(oh), ctypes.c_int64(1), ctypes.c_float(case["min"]),
                                                  ctypes.c_float(case["max"]), p(sc), p(sh), p(nl), p(nh)))
    np.testing.assert_allclose(sc[0], case["scale"], rtol=1e-6)
    np.testing.assert_allclose(sh[0], case["shift"], rtol=1e-6, atol=1e-6)
    assert nl[0] == case["min"] and nh[0] == case["max"]


def test_decompose_picks_precision_and_range():
    d = lpt.decompose_fake_quantize(256, np.float32(0), np.float32(2.55))
    assert d["precision"] == 40 and d["new_low"] == 0 and d["new_high"] == 255
    np.testing.assert_allclose(d["scale"], 0.01, rtol=1e-6)
    d = lpt.decompose_fake_quantize(256, np.float32(-1.28), np.float32(1.27))
    assert d["precision"] == 50 and d["new_low"] == -128 and d["new_high"] == 127
    with pytest.raises(NotImplementedError):
        lpt.decompose_fake_quantize(256, np.float32(0.12), np.float32(1.23))   # needs a zero point


@pytest.mark.parametrize("case", G["fold"]["cases"])
def test_fold_fake_quantize(case):
    v = np.array(case["values"], np.float32).reshape(2, 8)
    got = lpt.fold_fake_quantize(v, case["il"], case["ih"], case["ol"], case["oh"], case["levels"], case["round"])
    np.testing.assert_allclose(got.ravel(), np.array(case["expected"], np.float32), rtol=1e-5, atol=1e-5)


def test_convolution_weight_and_scale_golden():
    c = G["convolution"]
    d = lpt.decompose_fake_quantize(c["levels"], np.float32(c["ol"]), np.float32(c["oh"]))
    assert d["precision"] == 50 and (d["new_low"], d["new_high"]) == (-127, 127)
    q = lpt.fold_fake_quantize(np.array([[c["weight"]]], np.float32), c["il"], c["ih"], d["new_low"], d["new_high"],
                               c["levels"], True)
    assert q[0, 0] == c["expected_i8"]
    np.testing.assert_allclose(np.float32(c["act_scale"]) * d["scale"], c["expected_scale"], rtol=1e-6)
    m = G["matmul"]
    np.testing.assert_allclose(np.float32(m["scale_a"]) * np.float32(m["scale_b"]), m["expected"], rtol=1e-6)


def test_quantize_weights_roundtrip():
    rng = np.random.default_rng(0)
    w = rng.normal(0, 0.05, (8, 4, 3, 3)).astype(np.float32)
    q, s = lpt.quantize_weights(w)
    assert q.dtype == np.int8 and np.abs(q).max() == 127
    assert np.abs(q.astype(np.float32) * s.reshape(-1, 1, 1, 1) - w).max() <= s.max() / 2 + 1e-7


# ------------------------------------------------------------------ planner dry run (no device)
def _steps(g):
    from dldt_amd.graph import Plan
    return [(s["type"], s["name"]) for s in Plan(g, device=-1).steps]


def test_planner_fuses_resnet_block_chains():
    from dldt_amd import builders
    g, meta = builders.resnet50(batch=1, res=64, width=16, classes=10, seed=7)
    from dldt_amd.graph import Plan
    plan = Plan(g, device=-1)
    types = [s["type"] for s in plan.steps]
    # entry FQ, 53 convolutions (the 4 projection shortcuts run inside their residual convolution),
    # max-pool, avg-pool(+FQ), FC, exit; every elementwise node is fused away.  Seven bottleneck tails whose 3 x 3 layer
    # has 64 or 128 channels (stages 3 and 4 of this narrow net, without the blocks with a convolution in the shortcut)
    # are one step of two layers each
    assert types.count("Convolution,Convolution") == 7 and "Convolution+Convolution" not in types   # (no measurement in a dry run)
    assert types.count("Convolution") == 45 - 14 and types.count("Convolution+Shortcut") == 4
    assert types.count("MatMul") == 1 and types.count("MaxPool") == 1 and types.count("AvgPool") == 1
    assert types[0] == "FakeQuantize" and types[-1] == "Result" and len(types) == 54 - 7
    assert sum(int(plan.step_rt_info(i, "kernels")) for i in range(len(types))) == 54
    always = Plan(g, device=-1, config={"HIP_FUSE_CONVOLUTIONS": "YES"})
    assert [s["type"] for s in always.steps].count("Convolution+Convolution") == 7
    assert sum(int(always.step_rt_info(i, "kernels")) for i in range(len(always.steps))) == 47
    never = Plan(g, device=-1, config={"HIP_FUSE_CONVOLUTIONS": "NO"})
    assert len(never.steps) == 54 and always.config("HIP_FUSE_CONVOLUTIONS") == "YES" and plan.config("HIP_FUSE_CONVOLUTIONS") == "AUTO"
    assert sum(s["macs"] for s in plan.steps) == meta["macs_per_image"]
    assert plan.arena_bytes > 0
    with pytest.raises(Exception) as e:
        plan.create_request()
    assert "dry run" in str(e.value)


def test_planner_mobilenet_has_depthwise_steps():
    from dldt_amd import builders
    from dldt_amd.graph import Plan
    g, meta = builders.mobilenet_v2(batch=1, res=64, width=0.5, classes=10, last=128, seed=3)
    plan = Plan(g, device=-1)
    types = [s["type"] for s in plan.steps]
    assert types.count("GroupConvolution") == 17
    assert sum(s["macs"] for s in plan.steps) == meta["macs_per_image"]


def test_full_size_mac_counts_match_the_published_architecture():
    from dldt_amd import builders
    assert builders.resnet50_macs() == 4089184256          # 4.089 GMAC per image
    assert 0.29e9 < builders.mobilenet_v2(batch=1, res=224)[1]["macs_per_image"] < 0.32e9


def test_planner_encoder_stack_steps_and_views(monkeypatch):
    """BERT-style encoder: head split / merge are views (no step), the V operand gets one physical
    transpose, LayerNorm's Multiply and Add and the next FakeQuantize ride in the MVN step, and the published operation count of
    config 5 comes out: 565.3 GMAC for 12 layers at batch 16 x 384 tokens."""
    from dldt_amd import builders
    from dldt_amd.graph import Plan
    g, meta = builders.bert_encoder(layers=2, hidden=128, heads=2, ffn=256, batch=2, seq=128, seed=7)
    plan = Plan(g, device=-1)
    types = [s["type"] for s in plan.steps]
    attention = ["MatMul", "Attention", "MatMul"]          # Q, K, V projections as one GEMM; the core; the output projection
    ffn = ["MVN+FakeQuantize", "MatMul", "MatMul"]         # Gelu and its FakeQuantize ride in the up projection
    # every activation FakeQuantize but the first rides in the kernel that produces its input
    assert types == ["FakeQuantize"] + attention + ffn + ["MVN+FakeQuantize"] + attention + ffn + ["MVN", "Result"]
    assert sum(s["macs"] for s in plan.steps) == meta["macs"]
    monkeypatch.setenv("HIPIE_FUSE_ATTENTION", "0")       # separate kernels: V gets one physical transpose
    types = [s["type"] for s in Plan(g, device=-1).steps]
    assert types[1:6] == ["MatMul", "MatMul", "Softmax+FakeQuantize", "Transpose", "MatMul"]
    monkeypatch.setenv("HIPIE_MERGE_LINEAR", "0")         # and one GEMM per MatMul node
    types = [s["type"] for s in Plan(g, device=-1).steps]
    assert types[1:8] == ["MatMul", "MatMul", "MatMul", "Softmax+FakeQuantize", "MatMul", "Transpose", "MatMul"]
    T, H, FF = 16 * 384, 768, 3072
    assert 12 * (T * (4 * H * H + 2 * H * FF) + 2 * 16 * 12 * 384 * 384 * 64) == 565_325_070_336


def test_planner_refuses_a_reshape_that_moves_bytes():
    from dldt_amd import HipieError
    from dldt_amd.graph import Graph
    g = Graph()
    x = g.parameter("x", (2, 64, 128))
    t = g.transpose(x, (0, 2, 1))
    g.result(g.reshape(t, (2, 128 * 64)), "y")
    with pytest.raises(HipieError) as e:
        g.compile(device=-1)
    assert e.value.status == -2 and "Reshape" in str(e.value)


def test_planner_flattened_feature_map_in_front_of_a_fully_connected_layer():
    """[N, C, H, W] bytes -> Reshape [N, C * H * W] -> MatMul: planned as the convolution with an H x W filter; anything
    else that would read the flattened value in the reference's [C][H][W] order is refused"""
    from dldt_amd import HipieError, builders
    rng = np.random.default_rng(3)
    rnd = lambda s, k: (rng.standard_normal(s, dtype=np.float32) * np.float32(k)).astype(np.float32)
    net = builders.QuantizedNet()
    g = net.g
    a0 = net.input("data", (2, 8, 9, 11), 1.0)
    a1 = net.conv(a0, rnd((16, 8, 3, 3), 0.1), rnd(16, 0.2), 2.0, strides=(2, 2), pads=(1, 1))
    flat = dict(a1, node=g.reshape(a1["node"], (2, 16 * 5 * 6)))
    g.result(net.conv_f32(flat, rnd((10, 480), 0.05), rnd(10, 0.2), matmul=True), "fc")
    plan = g.compile(device=-1)
    assert [s["type"] for s in plan.steps] == ["FakeQuantize", "Convolution", "MatMul", "Result"]
    assert plan.steps[2]["macs"] == 2 * 10 * 480 and plan.outputs[0]["shape"] == (2, 10)
    # the flattened levels as a result of their own: their order in memory is not the reference's
    net = builders.QuantizedNet()
    g = net.g
    a0 = net.input("data", (2, 8, 9, 11), 1.0)
    a1 = net.conv(a0, rnd((16, 8, 3, 3), 0.1), rnd(16, 0.2), 2.0, strides=(2, 2), pads=(1, 1))
    g.result(net.dequantize(dict(a1, node=g.reshape(a1["node"], (2, 480)))), "flat")
    with pytest.raises(HipieError) as e:
        g.compile(device=-1)
    assert e.value.status == -2 and "flattened" in str(e.value)


def test_planner_embedding_front_end():
    from dldt_amd import builders
    from dldt_amd.graph import Plan
    g, meta = builders.bert_encoder(layers=1, hidden=128, heads=2, ffn=256, batch=2, seq=64, seed=9, vocab=300)
    plan = Plan(g, device=-1)
    types = [s["type"] for s in plan.steps]
    assert types[:3] == ["Gather", "MVN+FakeQuantize", "MatMul"] and "FakeQuantize" not in types
    assert plan.inputs[0]["dtype"] == 70 and plan.inputs[0]["shape"] == (2, 64)


def test_decompose_with_zero_point_golden():
    """[-1.28, 1.27] on a layer that only takes u8: shift 128, scale 0.01
    (lp_transformations/fake_quantize_transformation.cpp:153-183); optimizeSubtract rounds half away from zero."""
    from dldt_amd import lpt
    d = lpt.decompose_fake_quantize(256, np.float32(-1.28), np.float32(1.27), precision=40)
    assert d["precision"] == 40 and d["has_zero_point"] and d["new_low"] == 0 and d["new_high"] == 255
    np.testing.assert_allclose(d["scale"], 0.01, rtol=1e-6)
    np.testing.assert_allclose(d["shift"], 128.0, rtol=1e-6)
    np.testing.assert_array_equal(lpt.round_zero_point([94.239, 155.5, 0.49, 2.5, -0.5]), [94, 156, 0, 3, -1])
    a = lpt.decompose_fake_quantize(256, np.float32(-0.5), np.float32(2.0), allow_zero_point=True)
    assert a["precision"] == 40 and a["has_zero_point"]
    np.testing.assert_allclose(a["shift"], 51.0, rtol=1e-6)          # (0 * 2 - 255 * -0.5) / 2.5


def test_planner_takes_integer_zero_points():
    from dldt_amd import HipieError, builders
    from dldt_amd.graph import Graph, Plan
    g, _, _ = builders.zero_point_net()
    assert [s["type"] for s in Plan(g, device=-1).steps] == ["FakeQuantize", "Convolution", "Convolution", "Result"]
    # a fractional zero point (Subtract not passed through optimizeSubtract) is refused by name
    bad = Graph()
    x = bad.parameter("x", (1, 16, 8, 8))
    q = bad.fake_quantize(x, -1.0, 2.0, 0.0, 255.0, 256, 40)
    s = bad.subtract(bad.convert(q, 10), bad.constant(np.float32(85.3).reshape(())))
    y = bad.convolution(s, bad.constant(np.ones((16, 16, 1, 1), np.int8), 50))
    bad.result(bad.multiply(y, bad.constant(np.float32(0.1).reshape(()))), "y")
    with pytest.raises(HipieError) as e:
        Plan(bad, device=-1)
    assert e.value.status == -2 and "zero point" in str(e.value)


@pytest.mark.parametrize("case", G["fuse_elementwise"]["cases"], ids=lambda c: c["name"].split(" (")[0])
def test_fuse_elementwise_golden(case):
    """FakeQuantizeTransformation::fuseElementwise against the ranges the reference's own test expects: the operations
    are absorbed one at a time, the one next to the FakeQuantize first"""
    kinds = {"multiply": lpt.MULTIPLY, "subtract": lpt.SUBTRACT, "add": lpt.ADD}
    lo = np.float32(G["fuse_elementwise"]["in_low"])
    hi = np.float32(G["fuse_elementwise"]["in_high"])
    got = (np.atleast_1d(lo), np.atleast_1d(hi))
    for kind, value in case["steps"]:
        got = lpt.fuse_elementwise(kinds[kind], got[0], got[1], np.array(value, np.float32))
        if got is None:
            break
    if case["new_low"] is None:
        assert got is None
    else:
        np.testing.assert_allclose(got[0], case["new_low"], rtol=1e-6, atol=1e-5)
        np.testing.assert_allclose(got[1], case["new_high"], rtol=1e-6, atol=1e-5)


@pytest.mark.parametrize("case", G["add_both_branches"]["cases"], ids=lambda c: c["at"].split(" ")[0])
def test_add_transformation_golden(case):
    sh, sc, after = lpt.add_both_branches(case["full"][0], case["full"][1], case["empty"][0], case["empty"][1])
    np.testing.assert_allclose([sh[0], sc[0]], case["new_full"], rtol=1e-6)
    assert after[0] == np.float32(case["after"])


def test_swap_multiply_and_add_guard_and_broadcast():
    """bi / ai per element with either side broadcast, and 0 where both are 0 (network_helper.cpp:245-258); the
    reference's tests hold no literal for this step: it is one IEEE division per element"""
    b = np.array([1.0, 0.0, -3.0, 0.0], np.float32)
    a = np.array([4.0, 0.0, 0.5, 2.0], np.float32)
    got = lpt.swap_multiply_and_add(b, a)
    np.testing.assert_array_equal(got, np.array([0.25, 0.0, -6.0, 0.0], np.float32))
    np.testing.assert_array_equal(lpt.swap_multiply_and_add(np.float32(3), a[[0, 2, 3]]), np.float32(3) / a[[0, 2, 3]])
    np.testing.assert_array_equal(lpt.swap_multiply_and_add(b, np.float32(0.1)), b / np.float32(0.1))


def test_clamp_bounds_move_in_front_of_the_dequantization():
    """clamp.cpp:71-89: bounds divided by the scale (swapped for a negative one), then shifted; ReLU6 behind a
    per-tensor scale of 0.02 clamps the levels at 0 .. 300"""
    assert lpt.clamp_bounds(0.0, 6.0, 0.02) == (0.0, 6.0 / 0.02)
    assert lpt.clamp_bounds(0.0, 10.0, 3.0, 128.0) == (128.0, 10.0 / 3.0 + 128.0)
    assert lpt.clamp_bounds(0.0, 10.0, -5.0, 128.0) == (10.0 / -5.0 + 128.0, 128.0)


def test_builders_derive_their_constants_through_these_steps():
    """the post-LPT graphs of the benchmark configurations take b / s and il / s, ih / s from the pinned entry points"""
    import inspect
    from dldt_amd import builders
    src = inspect.getsource(builders)
    assert "lpt.swap_multiply_and_add" in src and "lpt.fuse_elementwise" in src
    code = "\n".join(l.split("#")[0] for l in src.splitlines() if '"""' not in l)
    assert "b / s)" not in code and "/ s_x)" not in code and "/ s)" not in code
