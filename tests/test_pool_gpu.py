"""MaxPool / AvgPool on quantized NHWC tensors through the graph-level C ABI (hipie_graph_max_pool,
hipie_graph_avg_pool) against the oracle: the reference's own hand vectors
(ngraph/test/backend/max_pool.in.cpp, avg_pool.in.cpp, every 4-D case) and seeded u8 / i8 fuzz over
ceil_mode, include-pad, asymmetric pads and windows whose in-bounds values are all negative."""
import json
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))


def _cases(stem):
    with open(os.path.join(HERE, "golden", stem + ".json")) as f:
        return {k: t for k, t in json.load(f)["tests"].items() if len(t["in_shape"]) == 4}


def _pads(t):
    """explicit pads of a golden (SAME_* resolved as the op's shape inference does)"""
    pb, pe = list(t["pads_begin"]), list(t["pads_end"])
    auto = t.get("auto_pad")
    if auto:
        for i in range(2):
            total = max((t["out_shape"][2 + i] - 1) * t["strides"][i] + t["kernel"][i] - t["in_shape"][2 + i], 0)
            lo, hi = total // 2, total - total // 2
            pb[i], pe[i] = (lo, hi) if auto == "SAME_UPPER" else (hi, lo)
    return pb, pe


def _pool_graph(shape, signed, kind, kernel, strides, pb, pe, ceil, exclude_pad=True, preserve=False):
    """Parameter f32 -> FakeQuantize to 8-bit levels (the identity on integer inputs) -> pool -> dequantization"""
    from dldt_amd.graph import Graph
    from dldt_amd.tensor import F32, I8, U8
    g = Graph()
    x = g.parameter("x", shape)
    lo, hi = (-128.0, 127.0) if signed else (0.0, 255.0)
    q = g.fake_quantize(x, lo, hi, lo, hi, 256, out_dtype=I8 if signed else U8)
    if kind == "max":
        p = g.max_pool(q, kernel, strides, pb, pe, ceil_mode=ceil)
        y = g.multiply(g.convert(p, F32), g.constant(np.float32(0.5).reshape(1, 1, 1, 1)))
    else:
        # after LPT the AvgPool reads the levels themselves and declares an f32 result (avg_pool.cpp:36-45 moves the
        # dequantization behind it)
        if preserve:
            # ... unless what reads the pool is quantized as well: then the AvgPool keeps the 8-bit type ("precision
            # preserved") and the reference's integer instantiation rounds the mean to a level
            p = g.avg_pool(q, kernel, strides, pb, pe, exclude_pad=exclude_pad, ceil_mode=ceil, out_dtype=I8 if signed else U8)
            y = g.multiply(g.convert(p, F32), g.constant(np.float32(0.5).reshape(1, 1, 1, 1)))
        else:
            p = g.avg_pool(q, kernel, strides, pb, pe, exclude_pad=exclude_pad, ceil_mode=ceil, out_dtype=F32)
            y = p
    g.result(y, "y")
    return g, p


def _run(orc, g, x):
    from interp import evaluate
    want, _ = evaluate(orc, g.nodes, {"x": x})
    req = g.compile().create_request()
    (got,) = req.infer(x)
    return got, want["y"]


@pytest.mark.parametrize("name", sorted(_cases("max_pool")))
def test_max_pool_reference_vectors(orc, name):
    t = _cases("max_pool")[name]
    pb, pe = _pads(t)
    x = np.asarray(t["a"], np.float32).reshape(t["in_shape"])
    g, _ = _pool_graph(t["in_shape"], False, "max", t["kernel"], t["strides"], pb, pe, t.get("ceil", False))
    got, want = _run(orc, g, x)
    assert got.shape == tuple(t["out_shape"])
    np.testing.assert_array_equal(got, want)
    np.testing.assert_array_equal(got, 0.5 * np.asarray(t["result"], np.float32).reshape(t["out_shape"]))


@pytest.mark.parametrize("name", sorted(_cases("avg_pool")))
def test_avg_pool_reference_vectors(orc, name):
    t = _cases("avg_pool")[name]
    pb, pe = _pads(t)
    x = np.asarray(t["a"], np.float32).reshape(t["in_shape"])
    # the engine pools 8-bit levels: a vector with halves among its inputs is fed doubled (the mean is linear and
    # doubling is exact in binary floating point), and so is its expected result
    k = np.float32(1.0 if np.array_equal(x, np.rint(x)) else 2.0)
    assert np.array_equal(x * k, np.rint(x * k))
    g, _ = _pool_graph(t["in_shape"], False, "avg", t["kernel"], t["strides"], pb, pe, t.get("ceil", False), t["exclude_pad"])
    got, want = _run(orc, g, x * k)
    assert got.shape == tuple(t["out_shape"])
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))
    np.testing.assert_allclose(got, k * np.asarray(t["result"], np.float32).reshape(t["out_shape"]), rtol=1e-6, atol=0)


GEOMETRIES = [
    # kernel, strides, pads_begin, pads_end, ceil
    ((3, 3), (2, 2), (1, 1), (1, 1), False),     # the ResNet stem pool
    ((3, 3), (2, 2), (0, 0), (1, 1), True),
    ((3, 3), (1, 1), (1, 1), (1, 1), False),
    ((2, 2), (2, 2), (0, 0), (0, 0), True),
    ((3, 2), (2, 1), (1, 0), (0, 1), False),     # asymmetric pads, rectangular window
    ((5, 5), (3, 3), (2, 1), (1, 2), True),
    ((2, 3), (1, 2), (1, 2), (0, 0), True),
    ((7, 7), (1, 1), (0, 0), (0, 0), False),     # global pool of a 7 x 7 map
]


@pytest.mark.parametrize("signed", [False, True])
@pytest.mark.parametrize("geo", range(len(GEOMETRIES)))
def test_max_pool_fuzz(orc, geo, signed):
    kernel, strides, pb, pe, ceil = GEOMETRIES[geo]
    rng = np.random.default_rng(100 + geo)
    h, w = (7, 7) if kernel == (7, 7) else (13, 10)
    shape = (3, 40, h, w)                         # 40 channels: padded to 48 in the arena
    lo, hi = (-128, 128) if signed else (0, 256)
    x = rng.integers(lo, hi, shape).astype(np.float32)
    if signed:
        x[1] = -np.abs(x[1]) - 1.0                # an image whose every value is negative: padding must never win
        x[1] = np.maximum(x[1], -128.0)
    g, p = _pool_graph(shape, signed, "max", kernel, strides, pb, pe, ceil)
    got, want = _run(orc, g, x)
    np.testing.assert_array_equal(got, want)
    if signed:
        assert got[1].max() < 0


@pytest.mark.parametrize("signed", [False, True])
@pytest.mark.parametrize("exclude_pad", [True, False])
@pytest.mark.parametrize("geo", range(len(GEOMETRIES)))
def test_avg_pool_fuzz(orc, geo, exclude_pad, signed):
    kernel, strides, pb, pe, ceil = GEOMETRIES[geo]
    rng = np.random.default_rng(200 + geo)
    h, w = (7, 7) if kernel == (7, 7) else (13, 10)
    shape = (2, 24, h, w)
    lo, hi = (-128, 128) if signed else (0, 256)
    x = rng.integers(lo, hi, shape).astype(np.float32)
    g, _ = _pool_graph(shape, signed, "avg", kernel, strides, pb, pe, ceil, exclude_pad)
    got, want = _run(orc, g, x)
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("signed", [False, True])
@pytest.mark.parametrize("exclude_pad", [True, False])
@pytest.mark.parametrize("geo", range(len(GEOMETRIES)))
def test_precision_preserved_avg_pool(orc, geo, exclude_pad, signed):
    """AvgPool with a u8 / i8 result (avg_pool.hpp for T = uint8_t / int8_t): nearbyint of the mean, ties to even, with
    the window sum kept in the element type as the reference keeps it (small values in the first image: no sum wraps,
    the result is the rounded mean; full-range values in the second: sums beyond the type wrap exactly alike)"""
    kernel, strides, pb, pe, ceil = GEOMETRIES[geo]
    rng = np.random.default_rng(300 + geo)
    h, w = (7, 7) if kernel == (7, 7) else (13, 10)
    shape = (2, 24, h, w)
    lo, hi = (-128, 128) if signed else (0, 256)
    x = rng.integers(lo, hi, shape).astype(np.float32)
    small = 127 // (kernel[0] * kernel[1])
    x[0] = rng.integers(-small if signed else 0, small + 1, shape[1:]).astype(np.float32)
    g, p = _pool_graph(shape, signed, "avg", kernel, strides, pb, pe, ceil, exclude_pad, preserve=True)
    got, want = _run(orc, g, x)
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))
    assert len(np.unique(got)) > 2


def test_window_in_the_padding_alone_is_refused():
    """ceil_mode can place the last window behind the tensor's last cell: the reference has no value for it"""
    from dldt_amd import HipieError
    from dldt_amd.graph import Graph
    from dldt_amd.tensor import U8
    g = Graph()
    x = g.parameter("x", (1, 16, 4, 4))
    q = g.fake_quantize(x, 0.0, 255.0, 0.0, 255.0, 256, out_dtype=U8)
    with pytest.raises(HipieError):
        g.max_pool(q, (2, 2), (3, 3), (0, 0), (2, 2), ceil_mode=True)   # windows start at 0, 3, 6: the third is padding only


# ---- pooling of f32 values (a layer in front of the first FakeQuantize, or behind a layer left in f32) --------------------
def _f32_pool(orc, x, kind, kernel, strides, pb, pe, ceil, exclude_pad=True):
    from dldt_amd.graph import Graph
    from interp import evaluate
    g = Graph()
    p = g.parameter("x", x.shape)
    y = g.max_pool(p, kernel, strides, pb, pe, ceil_mode=ceil) if kind == "max" else \
        g.avg_pool(p, kernel, strides, pb, pe, exclude_pad=exclude_pad, ceil_mode=ceil)
    g.result(y, "y")
    want, _ = evaluate(orc, g.nodes, {"x": x})
    (got,) = g.compile().create_request().infer(x)
    return got, want["y"]


@pytest.mark.parametrize("name", sorted(_cases("max_pool")))
def test_max_pool_reference_vectors_in_f32(orc, name):
    """the reference's vectors as they stand: f32 in, f32 out, no quantization in between"""
    t = _cases("max_pool")[name]
    pb, pe = _pads(t)
    x = np.asarray(t["a"], np.float32).reshape(t["in_shape"])
    got, want = _f32_pool(orc, x, "max", t["kernel"], t["strides"], pb, pe, t.get("ceil", False))
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))
    np.testing.assert_array_equal(got, np.asarray(t["result"], np.float32).reshape(t["out_shape"]))


@pytest.mark.parametrize("name", sorted(_cases("avg_pool")))
def test_avg_pool_reference_vectors_in_f32(orc, name):
    t = _cases("avg_pool")[name]
    pb, pe = _pads(t)
    x = np.asarray(t["a"], np.float32).reshape(t["in_shape"])
    got, want = _f32_pool(orc, x, "avg", t["kernel"], t["strides"], pb, pe, t.get("ceil", False), t["exclude_pad"])
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))
    np.testing.assert_allclose(got, np.asarray(t["result"], np.float32).reshape(t["out_shape"]), rtol=1e-6, atol=0)


@pytest.mark.parametrize("kind,exclude_pad", [("max", True), ("avg", True), ("avg", False)])
@pytest.mark.parametrize("geo", range(len(GEOMETRIES)))
def test_f32_pool_fuzz(orc, geo, kind, exclude_pad):
    kernel, strides, pb, pe, ceil = GEOMETRIES[geo]
    rng = np.random.default_rng(400 + geo)
    h, w = (7, 7) if kernel == (7, 7) else (13, 10)
    x = rng.normal(-0.5, 2.0, (2, 11, h, w)).astype(np.float32)
    x[1] = -np.abs(x[1]) - np.float32(0.25)       # every value negative: padding must never win a maximum
    got, want = _f32_pool(orc, x, kind, kernel, strides, pb, pe, ceil, exclude_pad)
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))
    if kind == "max":
        assert got[1].max() < 0
