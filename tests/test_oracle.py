"""Pins the CPU checker (oracle/) before anything is compared against it:
  1. the reference's own known-answer vectors (tests/golden/*.json),
  2. the reference's header kernels compiled in place (oracle/_ref), on seeded random inputs,
  3. what the mathematics fixes: integer conv == int64 brute force, 1x1 conv == GEMM, box filter,
     matmul == numpy on integers, closed-form FakeQuantize levels, level idempotence.
"""
import json
import os

import numpy as np
import pytest

G = os.path.join(os.path.dirname(__file__), "golden")


def load(stem):
    return json.load(open(os.path.join(G, stem + ".json")))["tests"]


# ------------------------------------------------------------------ 1. reference goldens
@pytest.mark.parametrize("name", sorted(load("fake_quantize")))
def test_fake_quantize_golden(orc, name):
    t = load("fake_quantize")[name]
    x = np.arange(np.prod(t["data_shape"]), dtype=np.float32).reshape(t["data_shape"])
    b = [np.array(t[k]["data"], np.float32).reshape(t[k]["shape"])
         for k in ("input_low", "input_high", "output_low", "output_high")]
    got = orc.fake_quantize(x, *b, t["levels"], bcast_axis=t.get("pdpd_axis", -2))
    np.testing.assert_allclose(got.ravel(), np.array(t["expected"], np.float32), rtol=1e-6)


def _prelu_cases():
    # (two of the 38 tests build their slope in a loop instead of writing it out: no literal vector to take)
    return {k: v for k, v in load("prelu").items() if all(f in v for f in ("a", "slope", "out", "shape_a", "shape_slope"))}


@pytest.mark.parametrize("name", sorted(_prelu_cases()))
def test_prelu_golden(orc, name):
    """ngraph/test/backend/prelu.in.cpp: scalar slopes, one per channel ([C], [C, 1, 1], [1, C, 1, W]), one per column,
    whole tensors - the 1-D slope that names the channels against the 1-D slope that broadcasts along the last axis"""
    t = _prelu_cases()[name]
    a = np.array(t["a"], np.float32).reshape(t["shape_a"])
    slope = np.array(t["slope"], np.float32).reshape(t["shape_slope"])
    np.testing.assert_array_equal(orc.prelu(a, slope), np.array(t["out"], np.float32).reshape(t["shape_a"]))


def test_prelu_golden_count():
    assert len(_prelu_cases()) == 36


def test_activations_closed_forms(orc):
    """Sigmoid and Swish on the inputs of the reference's sigmoid.in.cpp / swish.in.cpp (which compute their expected
    values by formula) against scipy's expit in double, to rounding; HSwish and HSigmoid on the points their
    definition fixes without arithmetic: 0 at and below -3, the identity (one) at and above 3, hswish(1) = 4 / 6"""
    from scipy.special import expit
    x = np.array([1, 8, -8, 17, -0.5, -1, 0.4, -5.7, -6, 3, -0.9, 23, 5, 3.3, 0.1, 0.6, 20, -7, -5.3, 3.5, -9, 11, 0], np.float32)
    np.testing.assert_allclose(orc.sigmoid(x), expit(x.astype(np.float64)), rtol=2e-7, atol=0)
    for beta in (1.0, 0.6, 0.33):
        np.testing.assert_allclose(orc.swish(x, beta), x.astype(np.float64) * expit(x.astype(np.float64) * np.float64(np.float32(beta))), rtol=3e-7,
                                   atol=1e-12)
    pts = np.array([-1e30, -100, -3.0000002, -3, 3, 3.0000002, 100, 1e30], np.float32)
    np.testing.assert_array_equal(orc.hsigmoid(pts), np.array([0, 0, 0, 0, 1, 1, 1, 1], np.float32))
    np.testing.assert_array_equal(orc.hswish(pts)[:4], np.zeros(4, np.float32))
    np.testing.assert_array_equal(orc.hswish(pts)[4:], pts[4:] * np.float32(6) / np.float32(6))
    assert orc.hswish(np.float32([1]))[0] == np.float32(4) / np.float32(6)
    assert orc.hsigmoid(np.float32([0]))[0] == np.float32(0.5) and orc.hswish(np.float32([-0.0]))[0] == 0


def _conv_cases(stem):
    return {k: v for k, v in load(stem).items()
            if all(f in v for f in ("inputs", "filters", "outputs", "strides", "padding"))}


@pytest.mark.parametrize("name", sorted(_conv_cases("convolution")))
def test_convolution_golden(orc, name):
    t = _conv_cases("convolution")[name]
    x = np.array(t["inputs"], np.float32).reshape(t["inputs_shape"])
    f = np.array(t["filters"], np.float32).reshape(t["filter_shape"])
    got = orc.convolution(x, f, t["strides"], t["dilations"], t["padding"], t["padding"])
    assert list(got.shape) == t["outputs_shape"]
    np.testing.assert_array_equal(got.ravel(), np.array(t["outputs"], np.float32))
    # integer instantiation gives the same numbers (all goldens are small integers)
    goti = orc.convolution(x.astype(np.int32), f.astype(np.int32), t["strides"], t["dilations"],
                           t["padding"], t["padding"])
    np.testing.assert_array_equal(goti.ravel(), np.array(t["outputs"]).astype(np.int32))


def test_convolution_golden_count():
    assert len(_conv_cases("convolution")) >= 20


@pytest.mark.parametrize("name", sorted(_conv_cases("group_convolution")))
def test_group_convolution_golden(orc, name):
    t = _conv_cases("group_convolution")[name]
    x = np.array(t["inputs"], np.float32).reshape(t["inputs_shape"])
    f = np.array(t["filters"], np.float32).reshape(t["filter_shape"])
    got = orc.convolution(x, f, t["strides"], t["dilations"], t["padding"], t["padding"],
                          grouped=True)
    assert list(got.shape) == t["outputs_shape"]
    np.testing.assert_array_equal(got.ravel(), np.array(t["outputs"], np.float32))


@pytest.mark.parametrize("name", sorted(load("matmul")))
def test_matmul_golden(orc, name):
    t = load("matmul")[name]
    for dt in (np.float32, np.int32, np.int64):
        a = np.array(t["a"], dt).reshape(t["a_shape"])
        b = np.array(t["b"], dt).reshape(t["b_shape"])
        got = orc.matmul(a, b, t["ta"], t["tb"])
        assert list(got.shape) == t["out_shape"]
        np.testing.assert_array_equal(got.ravel(), np.array(t["expected"], dt))


def _pool_pads(t):
    """Explicit pads of a pooling golden (SAME_* resolved as the op's shape inference does)."""
    pb, pe = list(t["pads_begin"]), list(t["pads_end"])
    if "auto_pad" in t:
        for i in range(2):
            total = max((t["out_shape"][2 + i] - 1) * t["strides"][i] + t["kernel"][i]
                        - t["in_shape"][2 + i], 0)
            lo, hi = total // 2, total - total // 2
            pb[i], pe[i] = (lo, hi) if t["auto_pad"] == "SAME_UPPER" else (hi, lo)
    return pb, pe


def _pool_cases(stem):
    return {k: v for k, v in load(stem).items() if len(v.get("in_shape", [])) == 4}


@pytest.mark.parametrize("name", sorted(_pool_cases("max_pool")))
def test_max_pool_golden(orc, name):
    t = _pool_cases("max_pool")[name]
    x = np.array(t["a"], np.float32).reshape(t["in_shape"])
    pb, pe = _pool_pads(t)
    got = orc.max_pool(x, t["kernel"], t["strides"], pb, pe, out_shape=tuple(t["out_shape"]))
    np.testing.assert_array_equal(got.ravel(), np.array(t["result"], np.float32))


@pytest.mark.parametrize("name", sorted(_pool_cases("avg_pool")))
def test_avg_pool_golden(orc, name):
    t = _pool_cases("avg_pool")[name]
    x = np.array(t["a"], np.float32).reshape(t["in_shape"])
    pb, pe = _pool_pads(t)
    got = orc.avg_pool(x, t["kernel"], t["strides"], pb, pe, not t["exclude_pad"],
                       out_shape=tuple(t["out_shape"]))
    np.testing.assert_allclose(got.ravel(), np.array(t["result"], np.float32), rtol=1e-6)


# ------------------------------------------------------------------ 2. compiled reference
def _fq_inputs(rng, shape, bshape):
    x = rng.normal(0, 1.5, shape).astype(np.float32)
    il = rng.uniform(-2, -0.1, bshape).astype(np.float32)
    ih = rng.uniform(0.1, 2, bshape).astype(np.float32)
    return x, il, ih


@pytest.mark.parametrize("bshape", [(), (1, 6, 1, 1), (6, 1, 1), (2, 6, 5, 7)])
@pytest.mark.parametrize("levels", [2, 16, 255, 256])
def test_fake_quantize_vs_ref(orc, ref, bshape, levels):
    rng = np.random.default_rng(7 + levels)
    x, il, ih = _fq_inputs(rng, (2, 6, 5, 7), bshape)
    for ol, oh in ((np.float32(0), np.float32(levels - 1)), (il, ih),
                   (np.float32(-1.27), np.float32(1.27))):
        a = orc.fake_quantize(x, il, ih, ol, oh, levels)
        b = ref.fake_quantize(x, il, ih, ol, oh, levels)
        np.testing.assert_array_equal(a.view(np.uint32), b.view(np.uint32))


def test_fake_quantize_ties_vs_ref(orc, ref):
    """Tie-dense input: values placed exactly on and one ulp either side of level midpoints."""
    rng = np.random.default_rng(11)
    C = 8
    il = rng.uniform(-3, -1, (1, C, 1, 1)).astype(np.float32)
    ih = rng.uniform(1, 3, (1, C, 1, 1)).astype(np.float32)
    k = np.arange(255, dtype=np.float32) + 0.5
    mid = (il + (ih - il) * (k.reshape(1, 1, 1, -1) / 255)).astype(np.float32)
    x = np.concatenate([mid, np.nextafter(mid, np.float32(9)), np.nextafter(mid, np.float32(-9)),
                        np.broadcast_to(il, mid.shape), np.broadcast_to(ih, mid.shape)], axis=2)
    a = orc.fake_quantize(x, il, ih, np.float32(0), np.float32(255), 256)
    b = ref.fake_quantize(x, il, ih, np.float32(0), np.float32(255), 256)
    np.testing.assert_array_equal(a, b)


CONV_FUZZ = [
    # in_shape, f_shape, strides, dil, pb, pe
    ((2, 3, 9, 8), (4, 3, 3, 3), (1, 1), (1, 1), (1, 1), (1, 1)),
    ((1, 5, 11, 7), (6, 5, 3, 2), (2, 1), (1, 2), (0, 1), (2, 0)),
    ((2, 4, 12, 12), (3, 4, 1, 1), (2, 2), (1, 1), (0, 0), (0, 0)),
    ((1, 2, 15, 15), (2, 2, 7, 7), (2, 2), (1, 1), (3, 3), (3, 3)),
    ((2, 3, 10), (4, 3, 3), (1,), (2,), (2,), (1,)),
    ((1, 2, 5, 6, 4), (3, 2, 2, 3, 2), (1, 2, 1), (1, 1, 1), (1, 0, 1), (0, 1, 1)),
]


@pytest.mark.parametrize("case", CONV_FUZZ)
def test_convolution_vs_ref(orc, ref, case):
    ish, fsh, st, di, pb, pe = case
    rng = np.random.default_rng(3)
    xi = rng.integers(0, 256, ish).astype(np.int32)
    fi = rng.integers(-127, 128, fsh).astype(np.int32)
    np.testing.assert_array_equal(orc.convolution(xi, fi, st, di, pb, pe),
                                  ref.convolution(xi, fi, st, di, pb, pe))
    xf = rng.normal(size=ish).astype(np.float32)
    ff = rng.normal(size=fsh).astype(np.float32)
    a, b = orc.convolution(xf, ff, st, di, pb, pe), ref.convolution(xf, ff, st, di, pb, pe)
    np.testing.assert_array_equal(a.view(np.uint32), b.view(np.uint32))  # same summation order


@pytest.mark.parametrize("groups,cg,ocg", [(4, 1, 1), (2, 3, 2), (8, 1, 2)])
def test_group_convolution_vs_ref(orc, ref, groups, cg, ocg):
    rng = np.random.default_rng(5)
    x = rng.integers(0, 256, (2, groups * cg, 9, 10)).astype(np.int32)
    f = rng.integers(-127, 128, (groups, ocg, cg, 3, 3)).astype(np.int32)
    for st in ((1, 1), (2, 2)):
        np.testing.assert_array_equal(
            orc.convolution(x, f, st, (1, 1), (1, 1), (1, 1), grouped=True),
            ref.convolution(x, f, st, (1, 1), (1, 1), (1, 1), grouped=True))


@pytest.mark.parametrize("a_shape,b_shape,ta,tb", [
    ((5, 7), (7, 3), False, False), ((7, 5), (3, 7), True, True), ((2, 3, 5, 7), (7, 4), False, False),
    ((2, 1, 5, 7), (1, 3, 4, 7), False, True), ((7,), (7, 4), False, False), ((3, 5, 7), (7,), False, False),
    ((4, 7, 5), (4, 7, 6), True, False)])
def test_matmul_vs_ref(orc, ref, a_shape, b_shape, ta, tb):
    rng = np.random.default_rng(9)
    a = rng.integers(-128, 128, a_shape).astype(np.int32)
    b = rng.integers(-128, 128, b_shape).astype(np.int32)
    np.testing.assert_array_equal(orc.matmul(a, b, ta, tb), ref.matmul(a, b, ta, tb))
    af, bf = rng.normal(size=a_shape).astype(np.float32), rng.normal(size=b_shape).astype(np.float32)
    x, y = orc.matmul(af, bf, ta, tb), ref.matmul(af, bf, ta, tb)
    np.testing.assert_array_equal(x.view(np.uint32), y.view(np.uint32))


def test_elementwise_vs_ref(orc, ref):
    rng = np.random.default_rng(13)
    a = rng.normal(size=(2, 5, 4, 3)).astype(np.float32)
    for bshape in ((1, 5, 1, 1), (5, 1, 1), (), (2, 5, 4, 3), (4, 1)):
        b = rng.normal(size=bshape).astype(np.float32) + np.float32(2)
        for op in ("add", "subtract", "multiply", "divide"):
            x, y = getattr(orc, op)(a, b), getattr(ref, op)(a, b)
            np.testing.assert_array_equal(x.view(np.uint32), y.view(np.uint32))
    np.testing.assert_array_equal(orc.relu(a), ref.relu(a))
    np.testing.assert_array_equal(orc.clamp(a, 0.0, 0.6), ref.clamp(a, 0.0, 0.6))
    wide = (rng.normal(size=4096) * 4).astype(np.float32)
    for op in ("hswish", "hsigmoid"):
        np.testing.assert_array_equal(getattr(orc, op)(wide).view(np.uint32), getattr(ref, op)(wide).view(np.uint32), err_msg=op)
    np.testing.assert_allclose(orc.sigmoid(wide), ref.sigmoid(wide), rtol=2e-7)
    for beta in (1.0, 0.6):
        np.testing.assert_allclose(orc.swish(wide, beta), ref.swish(wide, beta), rtol=3e-7, atol=1e-12)
    for sshape in ((1,), (5,), (3,), (1, 5, 1, 1), (5, 1, 1), (2, 5, 4, 3), (4, 1)):
        slope = rng.normal(size=sshape).astype(np.float32)
        x, y = orc.prelu(a, slope), ref.prelu(a, slope)
        np.testing.assert_array_equal(x.view(np.uint32), y.view(np.uint32), err_msg=str(sshape))


@pytest.mark.parametrize("dt", [np.uint8, np.int8, np.float32, np.int32])
def test_max_pool_vs_ref(orc, ref, dt):
    rng = np.random.default_rng(17)
    x = rng.integers(-100 if dt != np.uint8 else 0, 120, (2, 3, 9, 11)).astype(dt)
    for k, s, pb, pe in (((3, 3), (2, 2), (1, 1), (1, 1)), ((2, 3), (1, 2), (0, 1), (1, 0)),
                         ((9, 11), (1, 1), (0, 0), (0, 0))):
        np.testing.assert_array_equal(orc.max_pool(x, k, s, pb, pe), ref.max_pool(x, k, s, pb, pe))


@pytest.mark.parametrize("include_pad", [False, True])
def test_avg_pool_vs_ref(orc, ref, include_pad):
    rng = np.random.default_rng(19)
    xf = rng.normal(size=(2, 3, 7, 7)).astype(np.float32)
    xu = rng.integers(0, 256, (2, 3, 7, 7)).astype(np.uint8)
    for k, s, pb, pe in (((7, 7), (1, 1), (0, 0), (0, 0)), ((3, 3), (2, 2), (1, 1), (1, 1)),
                         ((2, 2), (1, 1), (0, 1), (1, 0))):
        a, b = orc.avg_pool(xf, k, s, pb, pe, include_pad), ref.avg_pool(xf, k, s, pb, pe, include_pad)
        np.testing.assert_array_equal(a.view(np.uint32), b.view(np.uint32))
        np.testing.assert_array_equal(orc.avg_pool(xu, k, s, pb, pe, include_pad),
                                      ref.avg_pool(xu, k, s, pb, pe, include_pad))
        xi = (xu.astype(np.int16) - 128).astype(np.int8)      # (sums that leave the int8 range included: the reference keeps them modulo 256)
        np.testing.assert_array_equal(orc.avg_pool(xi, k, s, pb, pe, include_pad),
                                      ref.avg_pool(xi, k, s, pb, pe, include_pad))


def test_fp32_glue_vs_ref(orc, ref):
    rng = np.random.default_rng(23)
    x = (rng.normal(size=(3, 4, 16, 33)) * 3).astype(np.float32)
    np.testing.assert_allclose(orc.softmax(x, -1), ref.softmax(x, -1), rtol=2e-6, atol=1e-9)
    y = x.reshape(-1, 33)
    for inside in (True, False):
        np.testing.assert_allclose(orc.mvn_last_axis(y, True, 1e-5, inside),
                                   ref.mvn_last_axis(y, True, 1e-5, inside), rtol=2e-6, atol=1e-7)
    np.testing.assert_allclose(orc.gelu_erf(x), ref.gelu_erf(x), rtol=1e-6, atol=1e-9)


# ------------------------------------------------------------------ 3. mathematics
def test_convolution_int_bruteforce(orc):
    rng = np.random.default_rng(29)
    N, C, H, W, OC, KH, KW, s, p, d = 2, 3, 7, 6, 4, 3, 2, 2, 1, 1
    x = rng.integers(0, 256, (N, C, H, W)).astype(np.int64)
    f = rng.integers(-127, 128, (OC, C, KH, KW)).astype(np.int64)
    OH, OW = (H + 2 * p - KH) // s + 1, (W + 2 * p - KW) // s + 1
    want = np.zeros((N, OC, OH, OW), np.int64)
    xp = np.pad(x, ((0, 0), (0, 0), (p, p), (p, p)))
    for oy in range(OH):
        for ox in range(OW):
            patch = xp[:, :, oy * s:oy * s + KH, ox * s:ox * s + KW]
            want[:, :, oy, ox] = np.einsum("nchw,ochw->no", patch, f)
    got = orc.convolution(x.astype(np.int32), f.astype(np.int32), (s, s), (d, d), (p, p), (p, p))
    np.testing.assert_array_equal(got, want.astype(np.int32))


def test_convolution_1x1_is_gemm_and_box(orc):
    rng = np.random.default_rng(31)
    x = rng.integers(0, 256, (2, 16, 5, 5)).astype(np.int32)
    f = rng.integers(-127, 128, (8, 16, 1, 1)).astype(np.int32)
    got = orc.convolution(x, f, (1, 1), (1, 1), (0, 0), (0, 0))
    want = np.einsum("nchw,oc->nohw", x, f[:, :, 0, 0])
    np.testing.assert_array_equal(got, want)
    ones = np.ones((1, 1, 6, 6), np.int32)
    box = orc.convolution(ones, np.ones((1, 1, 3, 3), np.int32), (1, 1), (1, 1), (1, 1), (1, 1))
    assert box[0, 0, 2, 2] == 9 and box[0, 0, 0, 0] == 4 and box[0, 0, 0, 3] == 6


def test_matmul_is_numpy(orc):
    rng = np.random.default_rng(37)
    a = rng.integers(-128, 128, (3, 2, 9, 17)).astype(np.int32)
    b = rng.integers(-128, 128, (2, 17, 5)).astype(np.int32)
    np.testing.assert_array_equal(orc.matmul(a, b), np.matmul(a, b))
    np.testing.assert_array_equal(orc.matmul(a, np.swapaxes(b, -1, -2), False, True), np.matmul(a, b))


def test_fake_quantize_closed_form(orc):
    """il=0, ih=2.55, L=256, out 0..255: level == rne(fl(fl(x/2.55)*255)) clamped to 0..255."""
    rng = np.random.default_rng(41)
    x = rng.uniform(-0.5, 3.0, 100000).astype(np.float32)
    got = orc.fake_quantize(x, np.float32(0), np.float32(2.55), np.float32(0), np.float32(255), 256)
    q = (x / np.float32(2.55)).astype(np.float32) * np.float32(255)
    want = np.where(x <= 0, 0, np.where(x > np.float32(2.55), 255, np.rint(q))).astype(np.float32)
    np.testing.assert_array_equal(got, want)
    assert set(np.unique(got)) <= set(np.arange(256, dtype=np.float32))
    # monotone in x
    xs = np.sort(x)
    ys = orc.fake_quantize(xs, np.float32(0), np.float32(2.55), np.float32(0), np.float32(255), 256)
    assert np.all(np.diff(ys) >= 0)


def test_fake_quantize_idempotent_on_levels(orc):
    """Re-quantising the op's own f32 outputs returns them unchanged."""
    il, ih = np.float32(-1.28), np.float32(1.27)
    x = np.linspace(-2, 2, 5001, dtype=np.float32)
    y = orc.fake_quantize(x, il, ih, il, ih, 256)
    z = orc.fake_quantize(y, il, ih, il, ih, 256)
    np.testing.assert_array_equal(y, z)
    assert len(np.unique(y)) == 256


def test_softmax_gelu_closed_forms(orc):
    from scipy import special
    rng = np.random.default_rng(43)
    x = rng.normal(size=(4, 37)).astype(np.float32) * 4
    np.testing.assert_allclose(orc.softmax(x, 1), special.softmax(x.astype(np.float64), 1), rtol=1e-5)
    np.testing.assert_allclose(orc.gelu_erf(x), 0.5 * x * (1 + special.erf(x / np.sqrt(2.0))),
                               rtol=1e-6, atol=1e-8)
    m = orc.mvn_last_axis(x, True, 1e-9, True)
    np.testing.assert_allclose(m.mean(1), 0, atol=1e-6)
    np.testing.assert_allclose(m.std(1), 1, rtol=1e-4)
