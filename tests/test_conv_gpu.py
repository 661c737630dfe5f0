"""Convolution on int8 MFMA through the C ABI vs the oracle: exact i32 accumulators and
bit-exact fused epilogues (bias, dequant scale, residual add, ReLU/Clamp, per-channel FQ)."""
import zlib

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

F32, I8, I32, U8B = 10, 50, 70, 41

# name: (N, C, H, W, OC, KH, KW, strides, dilations, pads_begin, pads_end)
GEOMS = {
    "3x3_s1_p1_c64": (2, 64, 14, 14, 64, 3, 3, (1, 1), (1, 1), (1, 1), (1, 1)),
    "1x1_c256_oc64": (2, 256, 7, 9, 64, 1, 1, (1, 1), (1, 1), (0, 0), (0, 0)),
    "1x1_c64_oc256": (1, 64, 15, 15, 256, 1, 1, (1, 1), (1, 1), (0, 0), (0, 0)),
    "1x1_s2_c128_oc512": (2, 128, 14, 14, 512, 1, 1, (2, 2), (1, 1), (0, 0), (0, 0)),
    "3x3_s2_p1_c128": (2, 128, 13, 13, 128, 3, 3, (2, 2), (1, 1), (1, 1), (1, 1)),
    "7x7_s2_p3_c3": (2, 3, 32, 32, 64, 7, 7, (2, 2), (1, 1), (3, 3), (3, 3)),
    "3x3_d2_p2_c16_oc40": (1, 16, 11, 10, 40, 3, 3, (1, 1), (2, 2), (2, 2), (2, 2)),
    "3x2_asym_c32_oc200": (3, 32, 9, 8, 200, 3, 2, (1, 2), (1, 1), (0, 1), (2, 0)),
    "5x5_p2_c20_oc24": (1, 20, 8, 8, 24, 5, 5, (1, 1), (1, 1), (2, 2), (2, 2)),
}


def _inputs(rng, g, signed=False):
    N, C, H, W, OC, KH, KW = g[:7]
    if signed:
        x = rng.integers(-128, 128, (N, C, H, W)).astype(np.int32)
    else:
        x = rng.integers(0, 256, (N, C, H, W)).astype(np.int32)
    w = rng.integers(-127, 128, (OC, C, KH, KW)).astype(np.int32)
    return x, w


def _k_steps(g):
    """64-byte steps of the K loop for geometry g: K runs over (kh, kw, padded channels), a 4-byte pixel (up to four
    channels) has every filter row padded to 16 bytes instead"""
    C, KH, KW = g[1], g[5], g[6]
    if C <= 4:
        k = KH * (-(-KW * 4 // 16) * 16)
    else:
        k = KH * KW * (-(-C // 16) * 16)
    return -(-k // 64)


def _device_in(x, g, signed=False):
    from dldt_amd import DeviceTensor
    pb, pe = g[9], g[10]
    halo = max(max(pb), max(pe))
    cs = 4 if x.shape[1] <= 4 else None
    return DeviceTensor.from_nchw(x, I8 if signed else U8B, halo=halo, c_stride=cs)


@pytest.mark.parametrize("tile", [0, 1, 2, 3, 4, 5, 6, 7, 10, 11])
@pytest.mark.parametrize("name", sorted(GEOMS))
def test_conv_i32_accumulators_exact(orc, name, tile):
    import torch
    from dldt_amd import Convolution, DeviceTensor, HipieError
    g = GEOMS[name]
    rng = np.random.default_rng(zlib.crc32(name.encode()))
    x, w = _inputs(rng, g)
    want = orc.convolution(x, w, g[7], g[8], g[9], g[10])
    xin = _device_in(x, g)
    conv = Convolution(w.astype(np.int8), xin, g[7], g[8], g[9], g[10])
    try:
        conv.set_tile(tile)
    except HipieError as e:       # the variants that split K over two wave groups need an even number of K steps
        assert 6 <= tile <= 7 and e.status == -4 and _k_steps(g) % 2 == 1
        return                    # refused exactly where it should be: nothing to run
    assert not (6 <= tile <= 7 and _k_steps(g) % 2 == 1)
    out = DeviceTensor(want.shape[0], want.shape[2], want.shape[3], want.shape[1], I32)
    conv.run(xin, out)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out.to_nchw(), want)


def test_conv_i8_activations_exact(orc):
    from dldt_amd import Convolution, DeviceTensor
    g = GEOMS["3x3_s1_p1_c64"]
    rng = np.random.default_rng(77)
    x, w = _inputs(rng, g, signed=True)
    want = orc.convolution(x, w, g[7], g[8], g[9], g[10])
    xin = _device_in(x, g, signed=True)
    out = DeviceTensor(want.shape[0], want.shape[2], want.shape[3], want.shape[1], I32)
    Convolution(w.astype(np.int8), xin, g[7], g[8], g[9], g[10]).run(xin, out)
    np.testing.assert_array_equal(out.to_nchw(), want)


def test_conv_extreme_values_do_not_overflow(orc):
    """All-255 activations against all -127 / +127 weights at K = 4608 (the largest ResNet-50
    reduction): |acc| = 1.49e8 < 2^31 and must come back exactly."""
    from dldt_amd import Convolution, DeviceTensor
    x = np.full((1, 512, 5, 5), 255, np.int32)
    w = np.full((64, 512, 3, 3), -127, np.int32)
    w[::2] = 127
    want = orc.convolution(x, w, (1, 1), (1, 1), (1, 1), (1, 1))
    assert abs(int(want.min())) > 1.4e8
    xin = DeviceTensor.from_nchw(x, U8B, halo=1)
    out = DeviceTensor(1, 5, 5, 64, I32)
    Convolution(w.astype(np.int8), xin, pads_begin=(1, 1), pads_end=(1, 1)).run(xin, out)
    np.testing.assert_array_equal(out.to_nchw(), want)


def _chain(orc, acc, bias=None, scale=None, res=None, res_scale=None, act=None, clamp=None, fq=None):
    """The post-LPT elementwise chain evaluated with the oracle's reference ops, NCHW."""
    OC = acc.shape[1]
    bc = (1, OC, 1, 1)
    v = acc.astype(np.float32)                       # Convert i32 -> f32
    if bias is not None:
        v = orc.add(v, np.asarray(bias, np.float32).reshape(bc))
    if scale is not None:
        v = orc.multiply(v, np.asarray(scale, np.float32).reshape(bc))
    if res is not None:
        r = res.astype(np.float32)
        if res_scale is not None:
            r = orc.multiply(r, np.asarray(res_scale, np.float32).reshape(-1, 1, 1) if np.size(res_scale) > 1
                             else np.float32(res_scale))
        v = orc.add(v, r)
    if act == "relu":
        v = orc.relu(v)
    elif act == "clamp":
        v = orc.clamp(v, clamp[0], clamp[1])
    if fq is not None:
        levels, il, ih, ol, oh = fq
        v = orc.fake_quantize(v, np.asarray(il, np.float32).reshape(bc if np.size(il) > 1 else ()),
                              np.asarray(ih, np.float32).reshape(bc if np.size(ih) > 1 else ()),
                              np.float32(ol), np.float32(oh), levels)
    return v


@pytest.mark.parametrize("name", ["3x3_s1_p1_c64", "1x1_c64_oc256", "7x7_s2_p3_c3", "3x2_asym_c32_oc200"])
def test_conv_bias_requantize_u8(orc, name):
    """Steady-state ResNet layer: u8 -> Conv'(i8 W) -> +b'[c] -> FQ(0, ih'[c] -> 0..255) -> u8."""
    from dldt_amd import Convolution, DeviceTensor, make_epilogue
    g = GEOMS[name]
    rng = np.random.default_rng(5)
    x, w = _inputs(rng, g)
    w = (w // 4)
    OC = g[4]
    acc = orc.convolution(x, w, g[7], g[8], g[9], g[10])
    amax = np.abs(acc).max()
    bias = rng.normal(0, amax / 20, OC).astype(np.float32)
    ih = rng.uniform(0.3, 1.0, OC).astype(np.float32) * np.float32(amax)
    il = np.zeros(OC, np.float32)
    fq = (256, il, ih, 0.0, 255.0)
    want = _chain(orc, acc, bias=bias, fq=fq).astype(np.uint8)
    xin = _device_in(x, g)
    out = DeviceTensor(acc.shape[0], acc.shape[2], acc.shape[3], OC, U8B)
    Convolution(w.astype(np.int8), xin, g[7], g[8], g[9], g[10],
                make_epilogue(bias=bias, out_dtype=U8B, fq=fq)).run(xin, out)
    np.testing.assert_array_equal(out.to_nchw(), want)
    assert np.all(out.padded_channels() == 0)


def test_conv_nonzero_input_low_and_ties(orc):
    """FQ with il != 0 and bias chosen so that many outputs sit exactly on level boundaries."""
    from dldt_amd import Convolution, DeviceTensor, make_epilogue
    g = GEOMS["1x1_c256_oc64"]
    rng = np.random.default_rng(6)
    x, w = _inputs(rng, g)
    w = np.sign(w)
    OC = g[4]
    acc = orc.convolution(x, w, g[7], g[8], g[9], g[10])
    # integer accumulators + half-integer bias against a range of width 255*2: x/2 lands on k+0.5
    bias = np.full(OC, 0.0, np.float32)
    il = np.full(OC, -255.0, np.float32)
    ih = np.full(OC, 255.0, np.float32)
    fq = (256, il, ih, 0.0, 255.0)
    want = _chain(orc, acc, bias=bias, fq=fq).astype(np.uint8)
    xin = _device_in(x, g)
    out = DeviceTensor(acc.shape[0], acc.shape[2], acc.shape[3], OC, U8B)
    Convolution(w.astype(np.int8), xin, g[7], g[8], g[9], g[10],
                make_epilogue(bias=bias, out_dtype=U8B, fq=fq)).run(xin, out)
    np.testing.assert_array_equal(out.to_nchw(), want)


_VARIANT_CASES = {}


def _variant_case(orc, kind):
    """One large layer per epilogue kind (enough pixel tiles that a persistent workgroup walks several),
    evaluated once by the oracle."""
    if kind in _VARIANT_CASES:
        return _VARIANT_CASES[kind]
    from dldt_amd import make_epilogue
    rng = np.random.default_rng(zlib.crc32(kind.encode()))
    if kind == "plain_3x3":
        g = (4, 16, 184, 184, 64, 3, 3, (1, 1), (1, 1), (1, 1), (1, 1))
    else:
        g = (4, 64, 184, 184, 64, 1, 1, (1, 1), (1, 1), (0, 0), (0, 0))
    x, w = _inputs(rng, g)
    OC = g[4]
    acc = orc.convolution(x, w, g[7], g[8], g[9], g[10])
    amax = np.float32(np.abs(acc).max())
    bias = rng.normal(0, amax / 20, OC).astype(np.float32)
    ih = rng.uniform(0.3, 1.0, OC).astype(np.float32) * amax
    res = None
    if kind in ("plain", "plain_3x3"):
        fq = (256, np.zeros(OC, np.float32), ih, 0.0, 255.0)
        want = _chain(orc, acc, bias=bias, fq=fq)
        epi = dict(bias=bias, out_dtype=U8B, fq=fq)
    elif kind == "plain_il":
        fq = (256, -ih / 3, ih, 0.0, 255.0)
        want = _chain(orc, acc, bias=bias, fq=fq)
        epi = dict(bias=bias, out_dtype=U8B, fq=fq)
    elif kind == "res_u8":
        scale = (rng.uniform(0.5, 2.0, OC) / amax).astype(np.float32)
        res = rng.integers(0, 256, acc.shape).astype(np.int32)
        s_x = rng.uniform(0.002, 0.004, OC).astype(np.float32)
        fq = (256, 0.0, np.float32(1.7), 0.0, 255.0)
        want = _chain(orc, acc, bias=bias, scale=scale, res=res, res_scale=s_x, fq=fq)
        epi = dict(bias=bias, scale=scale, residual_dtype=U8B, res_mul=s_x, out_dtype=U8B, fq=fq)
    else:   # "clamp": MobileNetV2 pointwise + ReLU6
        scale = (rng.uniform(2.0, 6.0, OC) / amax).astype(np.float32)
        fq = (256, 0.0, np.float32(6.0), 0.0, 255.0)
        want = _chain(orc, acc, bias=bias, scale=scale, act="clamp", clamp=(0.0, 6.0), fq=fq)
        epi = dict(bias=bias, scale=scale, activation="clamp", clamp=(0.0, 6.0), out_dtype=U8B, fq=fq)
    _VARIANT_CASES[kind] = (g, x, w, res, epi, want.astype(np.uint8))
    return _VARIANT_CASES[kind]


@pytest.mark.parametrize("tile", [0, 1, 4, 5, 8, 9, 10, 11])
@pytest.mark.parametrize("kind", ["plain", "plain_3x3", "plain_il", "res_u8", "clamp"])
def test_conv_kernel_variants_give_the_reference_bytes(orc, kind, tile):
    """Every kernel variant the tuner may pick, on layers of 135 424 pixels (529 or 1058 pixel tiles:
    the persistent variants walk several tiles per workgroup), against the oracle's fused chain."""
    from dldt_amd import Convolution, DeviceTensor, make_epilogue
    g, x, w, res, epi, want = _variant_case(orc, kind)
    xin = _device_in(x, g)
    conv = Convolution(w.astype(np.int8), xin, g[7], g[8], g[9], g[10], make_epilogue(**epi))
    conv.set_tile(tile)
    out = DeviceTensor(want.shape[0], want.shape[2], want.shape[3], want.shape[1], U8B)
    rt = DeviceTensor.from_nchw(res, U8B) if res is not None else None
    conv.run(xin, out, rt)
    np.testing.assert_array_equal(out.to_nchw(), want)


@pytest.mark.parametrize("res_kind", ["u8", "f32"])
def test_conv_residual_add_relu_requantize(orc, res_kind):
    """Bottleneck tail: (acc + b') * s[c] + residual -> ReLU -> FQ, residual either the u8 block
    input dequantised by a scalar (Convert, Multiply) or an f32 tensor (downsample branch)."""
    from dldt_amd import Convolution, DeviceTensor, make_epilogue
    g = GEOMS["1x1_c64_oc256"]
    rng = np.random.default_rng(8)
    x, w = _inputs(rng, g)
    OC = g[4]
    acc = orc.convolution(x, w, g[7], g[8], g[9], g[10])
    scale = (rng.uniform(0.5, 2.0, OC) * 1e-4).astype(np.float32)
    bias = rng.normal(0, 2000, OC).astype(np.float32)
    N, _, OH, OW = acc.shape
    fq = (256, 0.0, np.float32(6.0), 0.0, 255.0)
    xin = _device_in(x, g)
    out = DeviceTensor(N, OH, OW, OC, U8B)
    if res_kind == "u8":
        res = rng.integers(0, 256, acc.shape).astype(np.int32)
        s_x = np.float32(0.0173)
        want = _chain(orc, acc, bias=bias, scale=scale, res=res, res_scale=s_x, act="relu", fq=fq)
        rt = DeviceTensor.from_nchw(res, U8B)
        epi = make_epilogue(bias=bias, scale=scale, residual_dtype=U8B, res_mul=[s_x],
                            activation="relu", out_dtype=U8B, fq=fq)
    else:
        res = rng.normal(0, 3, acc.shape).astype(np.float32)
        want = _chain(orc, acc, bias=bias, scale=scale, res=res, act="relu", fq=fq)
        rt = DeviceTensor.from_nchw(res, F32)
        epi = make_epilogue(bias=bias, scale=scale, residual_dtype=F32, activation="relu",
                            out_dtype=U8B, fq=fq)
    Convolution(w.astype(np.int8), xin, g[7], g[8], g[9], g[10], epi).run(xin, out, rt)
    np.testing.assert_array_equal(out.to_nchw(), want.astype(np.uint8))


@pytest.mark.parametrize("act", [None, "relu", "clamp"])
def test_conv_dequantised_f32_output(orc, act):
    """Graph tail (benchmark configuration 1): Conv' -> +b' -> *s[c] -> ReLU, f32 out; bit-exact floats."""
    from dldt_amd import Convolution, DeviceTensor, make_epilogue
    g = GEOMS["3x3_s1_p1_c64"]
    rng = np.random.default_rng(10)
    x, w = _inputs(rng, g)
    OC = g[4]
    acc = orc.convolution(x, w, g[7], g[8], g[9], g[10])
    scale = (rng.uniform(0.5, 2.0, OC) * 1e-4).astype(np.float32)
    bias = rng.normal(0, 3000, OC).astype(np.float32)
    want = _chain(orc, acc, bias=bias, scale=scale, act=act, clamp=(0.0, 6.0))
    xin = _device_in(x, g)
    out = DeviceTensor(acc.shape[0], acc.shape[2], acc.shape[3], OC, F32)
    Convolution(w.astype(np.int8), xin, g[7], g[8], g[9], g[10],
                make_epilogue(bias=bias, scale=scale, activation=act, clamp=(0.0, 6.0),
                              out_dtype=F32)).run(xin, out)
    np.testing.assert_array_equal(out.to_nchw().view(np.uint32), want.view(np.uint32))


def test_conv_rejects_missing_halo_and_shape_mismatch():
    from dldt_amd import Convolution, DeviceTensor, HipieError
    w = np.ones((64, 64, 3, 3), np.int8)
    xin = DeviceTensor(1, 8, 8, 64, U8B, halo=0)
    conv = Convolution(w, xin, pads_begin=(1, 1), pads_end=(1, 1))
    with pytest.raises(HipieError) as e:
        conv.run(xin, DeviceTensor(1, 8, 8, 64, I32))
    assert e.value.status == -4 and "halo" in str(e.value)
    xin = DeviceTensor(1, 8, 8, 64, U8B, halo=1)
    conv = Convolution(w, xin, pads_begin=(1, 1), pads_end=(1, 1))
    with pytest.raises(HipieError):
        conv.run(xin, DeviceTensor(1, 7, 8, 64, I32))


@pytest.mark.parametrize("C,H,stride", [(32, 14, 1), (96, 15, 2), (144, 9, 1), (960, 7, 1)])
def test_depthwise_conv_exact_and_relu6_requantize(orc, C, H, stride):
    """MobileNetV2 depthwise 3x3 (GroupConvolution, G = C): i32 sums exact, then the post-LPT tail
    Add(b') -> Multiply(s[c]) -> Clamp(0, 6) -> FQ(0, 6 -> u8) bit-exact."""
    from dldt_amd import Convolution, DeviceTensor, make_epilogue
    rng = np.random.default_rng(C)
    x = rng.integers(0, 256, (2, C, H, H)).astype(np.int32)
    w = rng.integers(-127, 128, (C, 1, 1, 3, 3)).astype(np.int32)
    st = (stride, stride)
    acc = orc.convolution(x, w, st, (1, 1), (1, 1), (1, 1), grouped=True)
    xin = DeviceTensor.from_nchw(x, U8B, halo=1)
    N, _, OH, OW = acc.shape
    out = DeviceTensor(N, OH, OW, C, I32)
    Convolution(w.astype(np.int8), xin, st, (1, 1), (1, 1), (1, 1)).run(xin, out)
    np.testing.assert_array_equal(out.to_nchw(), acc)
    scale = (rng.uniform(0.5, 2.0, C) * 2e-4).astype(np.float32)
    bias = rng.normal(0, 3000, C).astype(np.float32)
    fq = (256, 0.0, np.float32(6.0), 0.0, 255.0)
    want = _chain(orc, acc, bias=bias, scale=scale, act="clamp", clamp=(0.0, 6.0), fq=fq).astype(np.uint8)
    out8 = DeviceTensor(N, OH, OW, C, U8B)
    Convolution(w.astype(np.int8), xin, st, (1, 1), (1, 1), (1, 1),
                make_epilogue(bias=bias, scale=scale, activation="clamp", clamp=(0.0, 6.0), out_dtype=U8B,
                              fq=fq)).run(xin, out8)
    np.testing.assert_array_equal(out8.to_nchw(), want)


DW_STRIP_GEOMS = [
    # N, C, H, W, stride, pads_begin, pads_end
    (2, 144, 56, 56, 1, (1, 1), (1, 1)),      # MobileNetV2 stage shapes
    (2, 144, 56, 56, 2, (1, 1), (1, 1)),
    (1, 32, 112, 112, 1, (1, 1), (1, 1)),
    (1, 96, 112, 112, 2, (1, 1), (1, 1)),
    (2, 192, 28, 28, 1, (1, 1), (1, 1)),
    (2, 384, 14, 14, 1, (1, 1), (1, 1)),
    (2, 576, 14, 14, 2, (1, 1), (1, 1)),
    (3, 960, 7, 7, 1, (1, 1), (1, 1)),
    (2, 48, 15, 11, 1, (1, 1), (1, 1)),       # ragged: rows not a multiple of 7, columns not of 4, 3 pixels' worth of lanes idle
    (2, 80, 9, 13, 2, (0, 0), (1, 1)),        # padding on the far sides only
    (1, 16, 5, 3, 1, (1, 1), (1, 1)),         # one strip wider than the row
    (1, 1008, 8, 6, 1, (1, 1), (1, 1)),       # 252 lanes of 256
]


@pytest.mark.parametrize("tail", ["clamp_fq", "scale_fq", "bias_fq"])
@pytest.mark.parametrize("geo", range(len(DW_STRIP_GEOMS)))
def test_depthwise_strip_variant_exact(orc, geo, tail):
    """the depthwise variant that stages its input in LDS and slides the window in registers gives the reference's
    levels bit for bit, for every FakeQuantize tail the depthwise kernels are specialised for"""
    from dldt_amd import Convolution, DeviceTensor, make_epilogue
    N, C, H, W, stride, pb, pe = DW_STRIP_GEOMS[geo]
    rng = np.random.default_rng(900 + geo)
    x = rng.integers(0, 256, (N, C, H, W)).astype(np.int32)
    w = rng.integers(-127, 128, (C, 1, 1, 3, 3)).astype(np.int32)
    st = (stride, stride)
    acc = orc.convolution(x, w, st, (1, 1), pb, pe, grouped=True)
    xin = DeviceTensor.from_nchw(x, U8B, halo=1)
    _, _, OH, OW = acc.shape
    bias = rng.normal(0, 3000, C).astype(np.float32)
    if tail == "clamp_fq":      # the Clamp is narrower than the FakeQuantize's range: it stays in the kernel
        scale = (rng.uniform(0.5, 2.0, C) * 2e-4).astype(np.float32)
        fq = (256, 0.0, np.float32(8.0), 0.0, 255.0)
        kw = dict(bias=bias, scale=scale, activation="clamp", clamp=(0.0, 6.0), fq=fq)
        want = _chain(orc, acc, bias=bias, scale=scale, act="clamp", clamp=(0.0, 6.0), fq=fq)
    elif tail == "scale_fq":    # ReLU6 in front of FQ(0, 6): the Clamp is implied by the FakeQuantize
        scale = (rng.uniform(0.5, 2.0, C) * 2e-4).astype(np.float32)
        fq = (256, 0.0, np.float32(6.0), 0.0, 255.0)
        kw = dict(bias=bias, scale=scale, activation="clamp", clamp=(0.0, 6.0), fq=fq)
        want = _chain(orc, acc, bias=bias, scale=scale, act="clamp", clamp=(0.0, 6.0), fq=fq)
    else:
        # per-channel divisors; a divisor without two-operation division constants sends the layer to the general
        # kernel (no variant 1), so draw until every channel's divisor has them
        from dldt_amd import HipieError
        for attempt in range(8):
            fq = (256, 0.0, rng.uniform(20000.0, 40000.0, C).astype(np.float32), 0.0, 255.0)
            kw = dict(bias=bias, fq=fq)
            probe = Convolution(w.astype(np.int8), xin, st, (1, 1), pb, pe, make_epilogue(out_dtype=U8B, **kw))
            try:
                probe.set_tile(1)
                break
            except HipieError:
                continue
        else:
            pytest.fail("no draw of divisors was accepted")
        want = _chain(orc, acc, bias=bias, fq=fq)
    want = want.astype(np.uint8)
    conv = Convolution(w.astype(np.int8), xin, st, (1, 1), pb, pe, make_epilogue(out_dtype=U8B, **kw))
    got = {}
    for variant in (0, 1, 2):
        if variant == 2 and pb != (1, 1):          # the matrix-pipe form is built for a padding of one on the top and left
            with pytest.raises(Exception):
                conv.set_tile(2)
            continue
        conv.set_tile(variant)
        assert conv.get_tile() == variant
        out8 = DeviceTensor(N, OH, OW, C, U8B)
        out8.interior().fill_(77)
        conv.run(xin, out8)
        got[variant] = out8.to_nchw()
        assert np.all(out8.padded_channels() == 0), "variant %d" % variant
    for variant, levels in got.items():
        np.testing.assert_array_equal(levels, want, err_msg="variant %d" % variant)


@pytest.mark.parametrize("N,C,H,W,stride", [(2, 144, 9, 11, 1), (1, 16, 5, 3, 1), (3, 48, 13, 40, 2), (2, 96, 17, 17, 2),
                                            (1, 1008, 6, 5, 1), (2, 32, 35, 70, 1), (1, 2048, 4, 4, 1)])
def test_depthwise_variants_with_per_channel_zero_points(orc, N, C, H, W, stride):
    """both depthwise variants (registers, LDS strip) on an input with one zero point per channel: the same levels as
    the reference's chain, rows and columns that leave partial tiles"""
    from dldt_amd import Convolution, DeviceTensor, HipieError, make_epilogue
    rng = np.random.default_rng(C * 7 + H)
    x = rng.integers(0, 256, (N, C, H, W)).astype(np.int32)
    zp = rng.integers(0, 256, C).astype(np.int32)
    w = rng.integers(-127, 128, (C, 1, 1, 3, 3)).astype(np.int32)
    st = (stride, stride)
    acc = orc.convolution(x - zp.reshape(1, C, 1, 1), w, st, (1, 1), (1, 1), (1, 1), grouped=True)
    _, _, OH, OW = acc.shape
    xin = DeviceTensor.from_nchw(x, U8B, halo=1, fill_level=0)
    import torch
    pattern = torch.from_numpy((zp - 128).astype(np.int8)).to(xin.view.device)
    full = xin.view
    full[:, 0, :, :C] = pattern
    full[:, -1, :, :C] = pattern
    full[:, :, 0, :C] = pattern
    full[:, :, -1, :C] = pattern
    bias = rng.normal(0, 3000, C).astype(np.float32)
    scale = (rng.uniform(0.5, 2.0, C) * 2e-4).astype(np.float32)
    fq = (256, 0.0, np.float32(6.0), 0.0, 255.0)
    want = _chain(orc, acc, bias=bias, scale=scale, act="clamp", clamp=(0.0, 6.0), fq=fq).astype(np.uint8)
    conv = Convolution(w.astype(np.int8), xin, st, (1, 1), (1, 1), (1, 1),
                       make_epilogue(bias=bias, scale=scale, activation="clamp", clamp=(0.0, 6.0), out_dtype=U8B, fq=fq),
                       zero_point=zp)
    ran = []
    for variant in (0, 1, 2):
        try:
            conv.set_tile(variant)
        except HipieError:
            assert variant == 1 and C > 1024           # the strip kernel stops at pixels of 1024 bytes
            continue
        out8 = DeviceTensor(N, OH, OW, C, U8B)
        out8.interior().fill_(77)
        conv.run(xin, out8)
        np.testing.assert_array_equal(out8.to_nchw(), want, err_msg="variant %d" % variant)
        ran.append(variant)
    assert 0 in ran and 2 in ran and (1 in ran or C > 1024)


def test_depthwise_strip_variant_is_refused_where_it_does_not_apply():
    from dldt_amd import Convolution, DeviceTensor, HipieError, make_epilogue
    x = DeviceTensor(1, 9, 9, 32, U8B, halo=2)
    w5 = np.ones((32, 1, 1, 5, 5), np.int8)
    conv = Convolution(w5, x, (1, 1), (1, 1), (2, 2), (2, 2))      # raw sums, 5 x 5
    with pytest.raises(HipieError):
        conv.set_tile(1)
    w3 = np.ones((32, 1, 1, 3, 3), np.int8)
    conv = Convolution(w3, x, (1, 1), (2, 2), (2, 2), (2, 2),
                       make_epilogue(bias=np.zeros(32, np.float32), out_dtype=U8B, fq=(256, 0.0, np.float32(6.0), 0.0, 255.0)))
    with pytest.raises(HipieError):
        conv.set_tile(1)                                            # dilated
    conv.set_tile(0)
    conv = Convolution(w3, x, (1, 1), (1, 1), (1, 1), (1, 1))       # raw sums: the strip variant has no such tail
    with pytest.raises(HipieError):
        conv.set_tile(1)


@pytest.mark.parametrize("signed,zp", [(False, 0), (False, 37), (False, 255), (True, -128), (True, 5)])
@pytest.mark.parametrize("depthwise", [False, True])
def test_conv_input_zero_point(orc, signed, zp, depthwise):
    """(x - zero point) * w summed exactly, with padding applied behind the subtraction: the input
    tensor's halo holds the zero-point level"""
    from dldt_amd import Convolution, DeviceTensor
    rng = np.random.default_rng(zp + 1000 * signed + 7 * depthwise)
    N, C, H, W, OC = 2, 32, 9, 11, 32 if depthwise else 40
    x = rng.integers(-128 if signed else 0, 128 if signed else 256, (N, C, H, W)).astype(np.int32)
    w = rng.integers(-127, 128, (C, 1, 1, 3, 3) if depthwise else (OC, C, 3, 3)).astype(np.int32)
    want = orc.convolution(x - zp, w, (1, 1), (1, 1), (1, 1), (1, 1), grouped=depthwise)
    xin = DeviceTensor.from_nchw(x, I8 if signed else U8B, halo=1, fill_level=zp)
    conv = Convolution(w.astype(np.int8), xin, (1, 1), (1, 1), (1, 1), (1, 1), zero_point=zp)
    out = DeviceTensor(N, H, W, OC, I32)
    conv.run(xin, out)
    np.testing.assert_array_equal(out.to_nchw(), want)


@pytest.mark.parametrize("depthwise", [False, True])
@pytest.mark.parametrize("signed", [False, True])
def test_conv_per_channel_input_zero_points(orc, signed, depthwise):
    """(x - zero point[c]) * w with one level per input channel; the halo holds channel c's level in channel c"""
    from dldt_amd import Convolution, DeviceTensor
    rng = np.random.default_rng(70 + signed + 2 * depthwise)
    N, C, H, W, OC = 2, 32, 9, 11, 32 if depthwise else 40
    lo, hi = (-128, 128) if signed else (0, 256)
    x = rng.integers(lo, hi, (N, C, H, W)).astype(np.int32)
    zp = rng.integers(lo, hi, C).astype(np.int32)
    w = rng.integers(-127, 128, (C, 1, 1, 3, 3) if depthwise else (OC, C, 3, 3)).astype(np.int32)
    want = orc.convolution(x - zp.reshape(1, C, 1, 1), w, (1, 1), (1, 1), (1, 1), (1, 1), grouped=depthwise)
    xin = DeviceTensor.from_nchw(x, I8 if signed else U8B, halo=1, fill_level=0)
    # the border: every pixel of the halo holds the channels' zero points
    full = xin.view                                                # [N, H + 2, W + 2, cs] stored bytes
    stored = (zp - (0 if signed else 128)).astype(np.int8)
    import torch
    pattern = torch.from_numpy(stored).to(full.device)
    full[:, 0, :, :C] = pattern
    full[:, -1, :, :C] = pattern
    full[:, :, 0, :C] = pattern
    full[:, :, -1, :C] = pattern
    conv = Convolution(w.astype(np.int8), xin, (1, 1), (1, 1), (1, 1), (1, 1), zero_point=zp)
    out = DeviceTensor(N, H, W, OC, I32)
    conv.run(xin, out)
    np.testing.assert_array_equal(out.to_nchw(), want)


@pytest.mark.parametrize("G,icg,ocg", [(2, 16, 24), (4, 8, 8), (32, 4, 4), (3, 5, 7)])
def test_group_convolution_with_several_channels_per_group(orc, G, icg, ocg):
    """GroupConvolution that is not depthwise (ResNeXt-style cardinality): every group convolved on its own
    (group_convolution.hpp:78-144), i32 sums exact, with a zero point and padding"""
    from dldt_amd import Convolution, DeviceTensor
    rng = np.random.default_rng(G * 100 + icg)
    N, H, W = 2, 9, 10
    C, OC = G * icg, G * ocg
    x = rng.integers(0, 256, (N, C, H, W)).astype(np.int32)
    w = rng.integers(-127, 128, (G, ocg, icg, 3, 3)).astype(np.int32)
    zp = 21
    want = orc.convolution(x - zp, w, (2, 1), (1, 1), (1, 1), (1, 1), grouped=True)
    xin = DeviceTensor.from_nchw(x, U8B, halo=1, fill_level=zp)
    conv = Convolution(w.astype(np.int8), xin, (2, 1), (1, 1), (1, 1), (1, 1), zero_point=zp)
    out = DeviceTensor(N, want.shape[2], want.shape[3], OC, I32)
    conv.run(xin, out)
    np.testing.assert_array_equal(out.to_nchw(), want)


@pytest.mark.parametrize("tile", [1, 2])
@pytest.mark.parametrize("G,icg,ocg,k", [(32, 4, 4, 3), (16, 8, 8, 3), (4, 64, 64, 3), (2, 128, 128, 1), (3, 16, 64, 3), (8, 32, 32, 1)])
def test_group_convolution_in_its_own_form(orc, G, icg, ocg, k, tile):
    """groups whose input channels lie in 16-byte-aligned spans under tiles of 64 output channels (ResNeXt cardinalities:
    32 x 4, 16 x 8, 8 x 32; wide groups of 64 and 128 channels; 192 output channels, a ragged 128-channel tile): every
    tile multiplies the K bytes of its own groups only, with a K-offset table of its own.  Both tiled kernels with
    64-channel tiles, per-channel zero points, stride, padding; i32 sums exact against
    reference::group_convolution on widened inputs"""
    from dldt_amd import Convolution, DeviceTensor
    rng = np.random.default_rng(G * 1000 + icg * 10 + k)
    N, H, W = 2, 11, 9
    C, OC = G * icg, G * ocg
    x = rng.integers(0, 256, (N, C, H, W)).astype(np.int32)
    w = rng.integers(-127, 128, (G, ocg, icg, k, k)).astype(np.int32)
    zp = rng.integers(0, 256, C).astype(np.int32)
    pad = k // 2
    want = orc.convolution(x - zp.reshape(1, C, 1, 1), w, (1, 2), (1, 1), (pad, pad), (pad, pad), grouped=True)
    xin = DeviceTensor.from_nchw(x, U8B, halo=pad, fill_level=0)
    if pad:
        import torch
        full = xin.view
        pattern = torch.from_numpy((zp - 128).astype(np.int8)).to(full.device)
        full[:, 0, :, :C] = pattern
        full[:, -1, :, :C] = pattern
        full[:, :, 0, :C] = pattern
        full[:, :, -1, :C] = pattern
    conv = Convolution(w.astype(np.int8), xin, (1, 2), (1, 1), (pad, pad), (pad, pad), zero_point=zp)
    conv.set_tile(tile)
    assert conv.get_tile() == tile
    with pytest.raises(Exception):
        conv.set_tile(4)                  # the dense kernels do not know the per-tile tables
    out = DeviceTensor(N, want.shape[2], want.shape[3], OC, I32)
    conv.run(xin, out)
    np.testing.assert_array_equal(out.to_nchw(), want)


_WIDE_CASES = {}


@pytest.mark.parametrize("tile", [0, 1, 4, 5, 6, 7, 10, 11])
@pytest.mark.parametrize("kind", ["f32", "f32_res", "i8"])
def test_conv_variants_on_ragged_channel_tiles(orc, kind, tile):
    """320 output channels (two and a half 128-channel tiles, five of 64), 722 pixels (ragged
    in every tile shape), f32 results with and without a late f32 residual and signed i8 levels: the
    encoder GEMMs' epilogues, through every variant the tuner may pick for them."""
    import torch
    from dldt_amd import Convolution, DeviceTensor, make_epilogue
    g = (2, 256, 19, 19, 320, 1, 1, (1, 1), (1, 1), (0, 0), (0, 0))
    if kind not in _WIDE_CASES:
        rng = np.random.default_rng(zlib.crc32(kind.encode()) + 1)
        x, w = _inputs(rng, g, signed=True)
        acc = orc.convolution(x, w, g[7], g[8], g[9], g[10])
        OC = g[4]
        amax = np.float32(np.abs(acc).max())
        bias = rng.normal(0, amax / 20, OC).astype(np.float32)
        scale = (rng.uniform(0.5, 2.0, OC) / amax).astype(np.float32)
        res = None
        if kind == "f32":
            want, epi = _chain(orc, acc, bias=bias, scale=scale), dict(bias=bias, scale=scale, out_dtype=F32)
        elif kind == "f32_res":
            res = rng.normal(0, 1, acc.shape).astype(np.float32)
            want = _chain(orc, acc, bias=bias, scale=scale, res=res)
            epi = dict(bias=bias, scale=scale, residual_dtype=F32, out_dtype=F32)
        else:
            fq = (256, np.float32(-1.28), np.float32(1.27), -128.0, 127.0)
            want = _chain(orc, acc, bias=bias, scale=scale, fq=fq).astype(np.int8)
            epi = dict(bias=bias, scale=scale, out_dtype=I8, fq=fq)
        _WIDE_CASES[kind] = (x, w, res, epi, want)
    x, w, res, epi, want = _WIDE_CASES[kind]
    xin = _device_in(x, g, signed=True)
    conv = Convolution(w.astype(np.int8), xin, g[7], g[8], g[9], g[10], make_epilogue(**epi))
    conv.set_tile(tile)
    out = DeviceTensor(2, 19, 19, 320, epi["out_dtype"])
    rt = DeviceTensor.from_nchw(res, F32) if res is not None else None
    conv.run(xin, out, rt)
    torch.cuda.synchronize()
    got = out.to_nchw()
    if kind == "i8":
        np.testing.assert_array_equal(got.view(np.int8) if got.dtype == np.uint8 else got.astype(np.int8), want)
    else:
        np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))



_ROW_GEOMS = {
    "c64_56x56": (2, 64, 56, 56, 64),
    "c128_28x28_oc128": (3, 128, 28, 28, 128),
    "ragged_13x19_oc96": (2, 64, 13, 19, 96),
    "two_tiles_30x9_c192": (1, 192, 30, 9, 64),
    "one_row_tiles_5x120": (2, 64, 5, 120, 64),
    "too_wide_3x300": (1, 64, 3, 300, 64),          # no patch fits: the general kernel runs instead
}


@pytest.mark.parametrize("epi", ["i32", "fq", "res_u8"])
@pytest.mark.parametrize("name", sorted(_ROW_GEOMS))
def test_conv_row_tile_kernel(orc, name, epi):
    """tile 12: whole output rows per workgroup, the input patch and the nine weight slices staged once in
    LDS (3 x 3, stride 1, pad 1): ragged last tiles of an image, several channel tiles, several 64-channel
    input slices, rows of up to 120 pixels"""
    import torch
    from dldt_amd import Convolution, DeviceTensor, HipieError, make_epilogue
    N, C, H, W, OC = _ROW_GEOMS[name]
    g = (N, C, H, W, OC, 3, 3, (1, 1), (1, 1), (1, 1), (1, 1))
    rng = np.random.default_rng(zlib.crc32((name + epi).encode()))
    x, w = _inputs(rng, g)
    acc = orc.convolution(x, w, g[7], g[8], g[9], g[10])
    xin = _device_in(x, g)
    res = rt = None
    if epi == "i32":
        want, e, dt = acc, None, I32
    else:
        amax = np.float32(np.abs(acc).max())
        bias = rng.normal(0, amax / 20, OC).astype(np.float32)
        ih = rng.uniform(0.3, 1.0, OC).astype(np.float32) * amax
        dt = U8B
        if epi == "fq":
            fq = (256, np.zeros(OC, np.float32), ih, 0.0, 255.0)
            want = _chain(orc, acc, bias=bias, fq=fq).astype(np.uint8)
            e = make_epilogue(bias=bias, out_dtype=U8B, fq=fq)
        else:
            scale = (rng.uniform(0.5, 2.0, OC) / amax).astype(np.float32)
            res = rng.integers(0, 256, acc.shape).astype(np.int32)
            s_x = rng.uniform(0.002, 0.004, OC).astype(np.float32)
            fq = (256, 0.0, np.float32(1.7), 0.0, 255.0)
            want = _chain(orc, acc, bias=bias, scale=scale, res=res, res_scale=s_x, fq=fq).astype(np.uint8)
            e = make_epilogue(bias=bias, scale=scale, residual_dtype=U8B, res_mul=s_x, out_dtype=U8B, fq=fq)
            rt = DeviceTensor.from_nchw(res, U8B)
    conv = Convolution(w.astype(np.int8), xin, g[7], g[8], g[9], g[10], e) if e is not None else \
        Convolution(w.astype(np.int8), xin, g[7], g[8], g[9], g[10])
    conv.set_tile(12)
    out = DeviceTensor(N, H, W, OC, dt)
    conv.run(xin, out, rt)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out.to_nchw(), want)


def test_row_tile_kernel_refuses_other_geometries():
    from dldt_amd import Convolution, HipieError
    for name in ("1x1_c64_oc256", "7x7_s2_p3_c3"):
        g = GEOMS[name]
        x, w = _inputs(np.random.default_rng(0), g)
        conv = Convolution(w.astype(np.int8), _device_in(x, g), g[7], g[8], g[9], g[10])
        with pytest.raises(HipieError) as e:
            conv.set_tile(12)
        assert e.value.status == -4


@pytest.mark.parametrize("stages", [3, 4, 6, 8])
@pytest.mark.parametrize("tile", [4, 5, 6, 7])
@pytest.mark.parametrize("name", ["3x3_s1_p1_c64", "1x1_c64_oc256", "3x2_asym_c32_oc200", "3x3_s2_p1_c128"])
def test_conv_pipelined_ring_depths(orc, name, tile, stages):
    """every ring depth the pipelined kernels have a loop for (deeper ones than fit the LDS round down),
    over K loops of 1 to 18 steps: fewer steps than stages, the peeled last step, the drained tail"""
    import torch
    from dldt_amd import Convolution, DeviceTensor, HipieError
    g = GEOMS[name]
    rng = np.random.default_rng(zlib.crc32(name.encode()) + 7)
    x, w = _inputs(rng, g)
    want = orc.convolution(x, w, g[7], g[8], g[9], g[10])
    xin = _device_in(x, g)
    conv = Convolution(w.astype(np.int8), xin, g[7], g[8], g[9], g[10])
    try:
        conv.set_tile(tile, stages)
    except HipieError as e:       # the variants that split K over two wave groups need an even number of K steps
        assert 6 <= tile <= 7 and e.status == -4 and _k_steps(g) % 2 == 1
        return                    # refused exactly where it should be: nothing to run
    assert not (6 <= tile <= 7 and _k_steps(g) % 2 == 1)
    out = DeviceTensor(want.shape[0], want.shape[2], want.shape[3], want.shape[1], I32)
    conv.run(xin, out)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out.to_nchw(), want)


_STEM_GEOMS = {
    # (N, C, H, W, OC, KH, KW, strides, pads)
    "resnet_stem_32": (2, 3, 32, 32, 64, 7, 7, (2, 2), (3, 3)),
    "resnet_stem_rows_of_112": (1, 3, 20, 224, 64, 7, 7, (2, 2), (3, 3)),      # two output rows per tile
    "odd_rows_oc96": (2, 3, 26, 38, 96, 7, 7, (2, 2), (3, 3)),                  # 13 output rows: one tile per image; 1.5 channel tiles
    "6x6_s2_c4": (1, 4, 30, 22, 64, 6, 6, (2, 2), (2, 2)),
    "5x8_s4x2_c2": (2, 2, 33, 40, 32, 5, 8, (4, 2), (2, 3)),
}


@pytest.mark.parametrize("extra_halo", [4, 0])
@pytest.mark.parametrize("epi", ["i32", "fq"])
@pytest.mark.parametrize("name", sorted(_STEM_GEOMS))
def test_conv_first_layer_kernel(orc, name, epi, extra_halo):
    """tile 13: 4-byte pixels, whole output rows per workgroup, patch and weights staged once, one 32-byte
    K slice per filter row whose surplus bytes meet zero weights; with no more halo than the padding needs,
    a patch that would overhang it makes the general kernel run instead"""
    import torch
    from dldt_amd import Convolution, DeviceTensor, make_epilogue
    N, C, H, W, OC, KH, KW, st, pad = _STEM_GEOMS[name]
    g = (N, C, H, W, OC, KH, KW, st, (1, 1), pad, pad)
    rng = np.random.default_rng(zlib.crc32((name + epi).encode()))
    x, w = _inputs(rng, g)
    acc = orc.convolution(x, w, g[7], g[8], g[9], g[10])
    from dldt_amd import DeviceTensor as DT
    xin = DT.from_nchw(x, U8B, halo=max(pad) + extra_halo, c_stride=4)
    if epi == "i32":
        want, conv, dt = acc, Convolution(w.astype(np.int8), xin, g[7], g[8], g[9], g[10]), I32
    else:
        amax = np.float32(np.abs(acc).max())
        bias = rng.normal(0, amax / 20, OC).astype(np.float32)
        ih = rng.uniform(0.3, 1.0, OC).astype(np.float32) * amax
        fq = (256, np.zeros(OC, np.float32), ih, 0.0, 255.0)
        want = _chain(orc, acc, bias=bias, fq=fq).astype(np.uint8)
        conv, dt = Convolution(w.astype(np.int8), xin, g[7], g[8], g[9], g[10], make_epilogue(bias=bias, out_dtype=U8B, fq=fq)), U8B
    conv.set_tile(13)
    out = DeviceTensor(acc.shape[0], acc.shape[2], acc.shape[3], OC, dt)
    conv.run(xin, out)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out.to_nchw(), want)


_SPLIT_GEOMS = {
    # (N, C, H, W, OC, KH, KW, strides, dilations, pads_begin, pads_end)
    "3x3_c64_oc64": GEOMS["3x3_s1_p1_c64"],                                              # 9 K steps, 4 tiles
    "3x3_s2_c128": GEOMS["3x3_s2_p1_c128"],                                              # 18 K steps, ragged pixel tile
    "3x3_c96_oc200_7x7": (5, 96, 7, 7, 200, 3, 3, (1, 1), (1, 1), (1, 1), (1, 1)),       # 14 steps (13.5 padded), ragged both ways
    "1x1_c704_oc136": (3, 704, 9, 9, 136, 1, 1, (1, 1), (1, 1), (0, 0), (0, 0)),         # 11 steps: uneven parts
    "1x1_c2304_oc72_one_tile": (1, 2304, 5, 5, 72, 1, 1, (1, 1), (1, 1), (0, 0), (0, 0)),   # 36 steps, one tile, up to 16 parts
    "3x3_c64_many_tiles": (20, 64, 28, 28, 320, 3, 3, (1, 1), (1, 1), (1, 1), (1, 1)),   # 123 x 3 tiles x 4 parts: more workgroups than fit at once
}


@pytest.mark.parametrize("tile", [14, 15, 16, 17])
@pytest.mark.parametrize("epi", ["i32", "fq", "res_u8", "f32_res"])
@pytest.mark.parametrize("name", sorted(_SPLIT_GEOMS))
def test_conv_k_split_over_workgroups(orc, name, epi, tile):
    """tiles 14 to 17: the K loop of a 128 x 128 tile split over 2 / 4 / 8 / 16 workgroups, partial accumulators through
    a workspace, the last workgroup to arrive adds them and runs the epilogue.  Three launches in a row on
    one stream with fresh inputs each time: the workspace and its counters are reused, stale partial sums
    or a counter that is not back at zero would show.  "f32_res" stores f32 through the LDS staging space that
    also holds the drawn ticket."""
    import torch
    from dldt_amd import Convolution, DeviceTensor, HipieError, make_epilogue
    g = _SPLIT_GEOMS[name]
    N, C, H, W, OC = g[:5]
    rng = np.random.default_rng(zlib.crc32((name + epi).encode()) + tile)
    x, w = _inputs(rng, g)
    acc = orc.convolution(x, w, g[7], g[8], g[9], g[10])
    amax = np.float32(np.abs(acc).max())
    bias = rng.normal(0, amax / 20, OC).astype(np.float32)
    ih = rng.uniform(0.3, 1.0, OC).astype(np.float32) * amax
    e, dt, res, res_kw = None, I32, None, {}
    if epi == "fq":
        fq = (256, np.zeros(OC, np.float32), ih, 0.0, 255.0)
        chain = dict(bias=bias, fq=fq)
        e, dt = make_epilogue(bias=bias, out_dtype=U8B, fq=fq), U8B
    elif epi == "res_u8":
        scale = (rng.uniform(0.5, 2.0, OC) / amax).astype(np.float32)
        s_x = rng.uniform(0.002, 0.004, OC).astype(np.float32)
        fq = (256, 0.0, np.float32(1.7), 0.0, 255.0)
        chain = dict(bias=bias, scale=scale, res_scale=s_x, fq=fq)
        e, dt = make_epilogue(bias=bias, scale=scale, residual_dtype=U8B, res_mul=s_x, out_dtype=U8B, fq=fq), U8B
    elif epi == "f32_res":
        scale = (rng.uniform(0.5, 2.0, OC) / amax).astype(np.float32)
        chain = dict(bias=bias, scale=scale)
        e, dt = make_epilogue(bias=bias, scale=scale, residual_dtype=F32, out_dtype=F32), F32
    xin = _device_in(x, g)
    conv = Convolution(w.astype(np.int8), xin, g[7], g[8], g[9], g[10], e) if e is not None else \
        Convolution(w.astype(np.int8), xin, g[7], g[8], g[9], g[10])
    try:
        conv.set_tile(tile)
    except HipieError as err:      # fewer than two K steps per part
        assert err.status == -4 and _k_steps(g) < 2 * (2 << (tile - 14))
        return                     # refused exactly where it should be: nothing to run
    assert _k_steps(g) >= 2 * (2 << (tile - 14))
    out = DeviceTensor(acc.shape[0], acc.shape[2], acc.shape[3], OC, dt)
    for rep in range(3):
        if rep:
            x, _ = _inputs(rng, g)
            acc = orc.convolution(x, w, g[7], g[8], g[9], g[10])
            xin = _device_in(x, g)
        rt = None
        if epi == "i32":
            want = acc
        elif epi == "f32_res":
            res = rng.normal(0, 1, acc.shape).astype(np.float32)
            rt = DeviceTensor.from_nchw(res, F32)
            want = _chain(orc, acc, res=res, **chain)
        else:
            if epi == "res_u8":
                res = rng.integers(0, 256, acc.shape).astype(np.int32)
                rt = DeviceTensor.from_nchw(res, U8B)
                want = _chain(orc, acc, res=res, **chain).astype(np.uint8)
            else:
                want = _chain(orc, acc, **chain).astype(np.uint8)
        conv.run(xin, out, rt)
        torch.cuda.synchronize()
        got = out.to_nchw()
        if dt == F32:
            got, want = got.view(np.uint32), np.ascontiguousarray(want, np.float32).view(np.uint32)
        np.testing.assert_array_equal(got, want, err_msg="launch %d" % rep)


def test_conv_k_split_streams_have_own_workspace(orc):
    """two streams run the same split-K convolution on different inputs at the same time, twenty launches
    each: every stream has its own partial sums and counters"""
    import torch
    from dldt_amd import Convolution, DeviceTensor
    g = _SPLIT_GEOMS["3x3_c96_oc200_7x7"]
    rng = np.random.default_rng(99)
    x0, w = _inputs(rng, g)
    x1, _ = _inputs(rng, g)
    wants = [orc.convolution(x, w, g[7], g[8], g[9], g[10]) for x in (x0, x1)]
    xins = [_device_in(x, g) for x in (x0, x1)]
    conv = Convolution(w.astype(np.int8), xins[0], g[7], g[8], g[9], g[10])
    conv.set_tile(15)
    outs = [DeviceTensor(wt.shape[0], wt.shape[2], wt.shape[3], wt.shape[1], I32) for wt in wants]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    torch.cuda.synchronize()
    for _ in range(20):
        for i in range(2):
            with torch.cuda.stream(streams[i]):
                conv.run(xins[i], outs[i])
    torch.cuda.synchronize()
    for i in range(2):
        np.testing.assert_array_equal(outs[i].to_nchw(), wants[i])


# ---- cache-line kernels (tiles 18 - 22): 128-byte (64-byte) K steps through buffer loads that write LDS ----
LINE_GEOMS = {
    # name: geometry, what it covers
    "1x1_c128_oc128_one_step": (2, 128, 9, 9, 128, 1, 1, (1, 1), (1, 1), (0, 0), (0, 0)),          # one 128-byte step
    "1x1_c256_oc200": (3, 256, 13, 13, 200, 1, 1, (1, 1), (1, 1), (0, 0), (0, 0)),                  # two steps, ragged tiles
    "1x1_s2_c384_oc72": (2, 384, 14, 14, 72, 1, 1, (2, 2), (1, 1), (0, 0), (0, 0)),                 # three steps: the ring exactly full
    "3x3_s1_p1_c128": (2, 128, 12, 11, 256, 3, 3, (1, 1), (1, 1), (1, 1), (1, 1)),                  # nine steps, halo reads
    "3x3_s2_p1_c256_oc320": (2, 256, 13, 13, 320, 3, 3, (2, 2), (1, 1), (1, 1), (1, 1)),            # 18 steps, two and a half channel tiles
    "1x1_c1024_many_tiles": (20, 1024, 14, 14, 256, 1, 1, (1, 1), (1, 1), (0, 0), (0, 0)),          # 31 pixel tiles: the XCD-aware order
    "3x3_d2_p2_c128": (1, 128, 10, 9, 64, 3, 3, (1, 1), (2, 2), (2, 2), (2, 2)),                    # dilated taps
    "1x1_c64_oc64": (3, 64, 17, 17, 64, 1, 1, (1, 1), (1, 1), (0, 0), (0, 0)),                      # 64-byte steps only (tile 22)
    "3x3_c64_oc96": (2, 64, 15, 14, 96, 3, 3, (1, 1), (1, 1), (1, 1), (1, 1)),                      # 64-byte steps only (tile 22)
}


@pytest.mark.parametrize("tile", [18, 19, 20, 21, 22])
@pytest.mark.parametrize("name", sorted(LINE_GEOMS))
def test_conv_line_kernels_exact(orc, name, tile):
    """i32 accumulators and the fused bias + per-channel FakeQuantize bytes of every cache-line variant"""
    import torch
    from dldt_amd import Convolution, DeviceTensor, HipieError, make_epilogue
    g = LINE_GEOMS[name]
    rng = np.random.default_rng(zlib.crc32(name.encode()) + tile)
    x, w = _inputs(rng, g)
    want = orc.convolution(x, w, g[7], g[8], g[9], g[10])
    xin = _device_in(x, g)
    conv = Convolution(w.astype(np.int8), xin, g[7], g[8], g[9], g[10])
    step = 64 if tile == 22 else 128
    if g[1] % step:
        with pytest.raises(HipieError) as e:     # a K step must not straddle two filter taps
            conv.set_tile(tile)
        assert e.value.status == -4
        return
    conv.set_tile(tile)
    out = DeviceTensor(want.shape[0], want.shape[2], want.shape[3], want.shape[1], I32)
    conv.run(xin, out)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(out.to_nchw(), want)
    OC = g[4]
    amax = np.float32(np.abs(want).max())
    bias = rng.normal(0, amax / 20, OC).astype(np.float32)
    ih = rng.uniform(0.3, 1.0, OC).astype(np.float32) * amax
    fq = (256, np.zeros(OC, np.float32), ih, 0.0, 255.0)
    want8 = _chain(orc, want, bias=bias, fq=fq).astype(np.uint8)
    conv8 = Convolution(w.astype(np.int8), xin, g[7], g[8], g[9], g[10], make_epilogue(bias=bias, out_dtype=U8B, fq=fq))
    conv8.set_tile(tile)
    out8 = DeviceTensor(want.shape[0], want.shape[2], want.shape[3], OC, U8B)
    conv8.run(xin, out8)
    np.testing.assert_array_equal(out8.to_nchw(), want8)
    assert np.all(out8.padded_channels() == 0)


@pytest.mark.parametrize("tile", [18, 19, 22])
@pytest.mark.parametrize("kind", ["res_u8", "f32", "i8_signed_in"])
def test_conv_line_kernels_other_epilogues(orc, kind, tile):
    """u8 residual + requantisation, dequantised f32 output (staged stores), signed i8 activations"""
    from dldt_amd import Convolution, DeviceTensor, make_epilogue
    g = (3, 128, 14, 13, 320, 1, 1, (1, 1), (1, 1), (0, 0), (0, 0))
    rng = np.random.default_rng(zlib.crc32(kind.encode()) + tile)
    signed = kind == "i8_signed_in"
    x, w = _inputs(rng, g, signed=signed)
    OC = g[4]
    acc = orc.convolution(x, w, g[7], g[8], g[9], g[10])
    amax = np.float32(np.abs(acc).max())
    bias = rng.normal(0, amax / 20, OC).astype(np.float32)
    xin = _device_in(x, g, signed=signed)
    rt = None
    if kind == "res_u8":
        scale = (rng.uniform(0.5, 2.0, OC) / amax).astype(np.float32)
        res = rng.integers(0, 256, acc.shape).astype(np.int32)
        s_x = rng.uniform(0.002, 0.004, OC).astype(np.float32)
        fq = (256, 0.0, np.float32(1.7), 0.0, 255.0)
        want = _chain(orc, acc, bias=bias, scale=scale, res=res, res_scale=s_x, fq=fq).astype(np.uint8)
        epi = make_epilogue(bias=bias, scale=scale, residual_dtype=U8B, res_mul=s_x, out_dtype=U8B, fq=fq)
        rt = DeviceTensor.from_nchw(res, U8B)
        out = DeviceTensor(acc.shape[0], acc.shape[2], acc.shape[3], OC, U8B)
    else:
        scale = (rng.uniform(0.5, 2.0, OC) * 1e-4).astype(np.float32)
        want = _chain(orc, acc, bias=bias, scale=scale)
        epi = make_epilogue(bias=bias, scale=scale, out_dtype=F32)
        out = DeviceTensor(acc.shape[0], acc.shape[2], acc.shape[3], OC, F32)
    conv = Convolution(w.astype(np.int8), xin, g[7], g[8], g[9], g[10], epi)
    conv.set_tile(tile)
    conv.run(xin, out, rt)
    if kind == "res_u8":
        np.testing.assert_array_equal(out.to_nchw(), want)
    else:
        np.testing.assert_array_equal(out.to_nchw().view(np.uint32), want.view(np.uint32))
