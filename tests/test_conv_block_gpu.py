"""The patch-staged 3 x 3 kernel (variant 24) and the fused bottleneck tail (3 x 3 -> 1 x 1 with residual in one
launch, hipie_conv_run_pair) through the C ABI against the oracle: the same bytes as the node-by-node chain."""
import zlib

import numpy as np
import pytest

from test_conv_gpu import _chain, _inputs

pytestmark = pytest.mark.gpu

F32, I8, I32, U8B = 10, 50, 70, 41

# name: (N, C, H, W, OC of the 3 x 3 layer, OC of the 1 x 1 layer)
CASES = {
    "c64_14x14": (2, 64, 14, 14, 64, 256),            # one tile per image
    "c64_30x20_ragged": (2, 64, 30, 20, 64, 128),     # 12 + 12 + 6 rows
    "c64_56x56": (3, 64, 56, 56, 64, 256),            # ResNet-50 stage 1
    "c128_28x28": (5, 128, 28, 28, 128, 512),         # stage 2; 35 tiles: the XCD order leaves five blocks idle
    "c256_14x14": (2, 256, 14, 14, 256, 1024),        # stage 3: rows 4 + 4 + 4 + 2
    "c192_to_128_9x7": (1, 192, 9, 7, 128, 128),      # three input slabs, other channel count out, one pass
    "c64_to_256_5x5": (2, 64, 5, 5, 256, 256),        # a tile far smaller than its pixel slots
    "c128_to_256_20x12": (2, 128, 20, 12, 256, 512),  # two input slabs, two passes, rows 5 + 5 + 5 + 5
}
# the cases the form with two wave groups takes (an even number of input slabs, 128 or 256 channels between the layers)
TWO_GROUPS = ("c128_28x28", "c256_14x14", "c128_to_256_20x12")
ST, DIL, PAD = (1, 1), (1, 1), (1, 1)


def _first_layer(orc, rng, case):
    N, C, H, W, OC, _ = case
    x, w = _inputs(rng, (N, C, H, W, OC, 3, 3))
    w = w // 4
    acc = orc.convolution(x, w, ST, DIL, PAD, PAD)
    amax = np.float32(np.abs(acc).max())
    bias = rng.normal(0, amax / 20, OC).astype(np.float32)
    ih = rng.uniform(0.3, 1.0, OC).astype(np.float32) * amax
    fq = (256, np.zeros(OC, np.float32), ih, 0.0, 255.0)
    mid = _chain(orc, acc, bias=bias, fq=fq).astype(np.uint8)
    return x, w, dict(bias=bias, out_dtype=U8B, fq=fq), mid


@pytest.mark.parametrize("name", sorted(CASES))
def test_patch_staged_3x3_gives_the_reference_bytes(orc, name):
    from dldt_amd import Convolution, DeviceTensor, make_epilogue
    case = CASES[name]
    rng = np.random.default_rng(zlib.crc32(name.encode()))
    x, w, epi, want = _first_layer(orc, rng, case)
    xin = DeviceTensor.from_nchw(x, U8B, halo=1)
    conv = Convolution(w.astype(np.int8), xin, ST, DIL, PAD, PAD, make_epilogue(**epi))
    conv.set_tile(24)
    assert conv.get_tile() == 24
    out = DeviceTensor(want.shape[0], want.shape[2], want.shape[3], want.shape[1], U8B)
    conv.run(xin, out)
    np.testing.assert_array_equal(out.to_nchw(), want)
    assert np.all(out.padded_channels() == 0)


@pytest.mark.parametrize("name", sorted(CASES))
def test_fused_bottleneck_tail_gives_the_reference_bytes(orc, name):
    """3 x 3 (bias, FakeQuantize) -> 1 x 1 (bias, scale, u8 residual, FakeQuantize) in one kernel: the bytes of the
    oracle's chain, and of the two layers run one after the other."""
    from dldt_amd import Convolution, DeviceTensor, make_epilogue
    case = CASES[name]
    N, C, H, W, OCA, OCB = case
    rng = np.random.default_rng(zlib.crc32(name.encode()) + 1)
    x, w, epi_a, mid = _first_layer(orc, rng, case)
    w2 = rng.integers(-127, 128, (OCB, OCA, 1, 1)).astype(np.int32) // 2
    acc2 = orc.convolution(mid.astype(np.int32), w2, ST, DIL, (0, 0), (0, 0))
    amax = np.float32(np.abs(acc2).max())
    bias2 = rng.normal(0, amax / 20, OCB).astype(np.float32)
    scale2 = (rng.uniform(0.5, 2.0, OCB) / amax).astype(np.float32)
    res = rng.integers(0, 256, acc2.shape).astype(np.int32)
    s_x = rng.uniform(0.002, 0.004, OCB).astype(np.float32)
    fq2 = (256, 0.0, np.float32(1.7), 0.0, 255.0)
    want = _chain(orc, acc2, bias=bias2, scale=scale2, res=res, res_scale=s_x, fq=fq2).astype(np.uint8)

    xin = DeviceTensor.from_nchw(x, U8B, halo=1)
    tmid = DeviceTensor(N, H, W, OCA, U8B)
    first = Convolution(w.astype(np.int8), xin, ST, DIL, PAD, PAD, make_epilogue(**epi_a))
    second = Convolution(w2.astype(np.int8), tmid, ST, DIL, (0, 0), (0, 0),
                         make_epilogue(bias=bias2, scale=scale2, residual_dtype=U8B, res_mul=s_x, out_dtype=U8B, fq=fq2))
    rt = DeviceTensor.from_nchw(res, U8B)
    assert first.pair_fits(second, H, W)
    out = DeviceTensor(N, H, W, OCB, U8B)
    first.run_pair(second, xin, out, rt)
    np.testing.assert_array_equal(out.to_nchw(), want)
    assert np.all(out.padded_channels() == 0)
    # the other forms of the kernel: nine steps of weights in flight, and eight waves in two groups where it applies
    assert (first.pair_forms(second, H, W) & 2 != 0) == (name in TWO_GROUPS)
    for stages in (8, 7) if name in TWO_GROUPS else (8,):
        first.set_stages(stages)
        again = DeviceTensor(N, H, W, OCB, U8B)
        first.run_pair(second, xin, again, rt)
        np.testing.assert_array_equal(again.to_nchw(), want, err_msg="stages %d" % stages)
    if name not in TWO_GROUPS:
        first.set_stages(7)
        with pytest.raises(Exception):
            first.run_pair(second, xin, DeviceTensor(N, H, W, OCB, U8B), rt)
    first.set_stages(0)
    # the layers one after the other store the same bytes
    first.run(xin, tmid)
    np.testing.assert_array_equal(tmid.to_nchw(), mid)
    out2 = DeviceTensor(N, H, W, OCB, U8B)
    second.run(tmid, out2, rt)
    np.testing.assert_array_equal(out2.to_nchw(), want)


def test_pair_is_refused_where_the_kernel_does_not_apply():
    from dldt_amd import Convolution, DeviceTensor, HipieError, make_epilogue
    rng = np.random.default_rng(3)
    fq = (256, 0.0, np.float32(900.0), 0.0, 255.0)
    xin = DeviceTensor(1, 9, 9, 64, U8B, halo=1)
    w = rng.integers(-3, 4, (64, 64, 3, 3)).astype(np.int8)
    first = Convolution(w, xin, ST, DIL, PAD, PAD, make_epilogue(bias=np.zeros(64, np.float32), out_dtype=U8B, fq=fq))
    strided = Convolution(w, xin, (2, 2), DIL, PAD, PAD, make_epilogue(bias=np.zeros(64, np.float32), out_dtype=U8B, fq=fq))
    tmid = DeviceTensor(1, 9, 9, 64, U8B)
    w2 = rng.integers(-3, 4, (128, 64, 1, 1)).astype(np.int8)
    plain_second = Convolution(w2, tmid, epilogue=make_epilogue(bias=np.zeros(128, np.float32), out_dtype=U8B, fq=fq))
    assert not first.pair_fits(plain_second, 9, 9)        # no residual: not an epilogue the kernel is built for
    assert not strided.pair_fits(plain_second, 9, 9)
    with pytest.raises(HipieError) as e:
        first.run_pair(plain_second, xin, DeviceTensor(1, 9, 9, 128, U8B))
    assert e.value.status == -4
    with pytest.raises(HipieError):
        strided.set_tile(24)
