"""hipie_conv_run_static: the convolution entry point that allocates nothing (its K-split workspace is a fixed
device array inside the library) against hipie_conv_run, bit for bit, on two calls in a row - the second with a
smaller input - and its refusal of launches that the fixed array cannot hold."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

I32, U8B = 70, 41


def _case(rng, n, c, hw, oc, k):
    x = rng.integers(0, 256, (n, c, hw, hw)).astype(np.int32)
    w = rng.integers(-127, 128, (oc, c, k, k)).astype(np.int32)
    return x, w


@pytest.mark.parametrize("tile", [14, 15, 17])
def test_static_scratch_entry_point_matches_the_allocating_one(orc, tile):
    import torch
    from dldt_amd import Convolution, DeviceTensor, make_epilogue
    rng = np.random.default_rng(700 + tile)
    # first call: 14 tiles of 128 x 128 (two channel tiles); second call: a smaller batch, 4 tiles, other values
    for n in (4, 1):
        x, w = _case(rng, n, 2304, 14, 256, 1)
        xin = DeviceTensor.from_nchw(x, U8B)
        want = orc.convolution(x, w, (1, 1), (1, 1), (0, 0), (0, 0))
        conv = Convolution(w.astype(np.int8), xin)
        conv.set_tile(tile)
        ref = DeviceTensor(n, 14, 14, 256, I32)
        out = DeviceTensor(n, 14, 14, 256, I32)
        conv.run(xin, ref)
        conv.run_static(xin, out)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(out.to_nchw(), ref.to_nchw())
        np.testing.assert_array_equal(out.to_nchw(), want)
        # a fused epilogue through the same entry point (bias + per-channel FakeQuantize to u8 levels)
        amax = np.float32(np.abs(want).max())
        bias = rng.normal(0, amax / 20, 256).astype(np.float32)
        fq = (256, np.zeros(256, np.float32), rng.uniform(0.3, 1.0, 256).astype(np.float32) * amax, 0.0, 255.0)
        conv8 = Convolution(w.astype(np.int8), xin, epilogue=make_epilogue(bias=bias, out_dtype=U8B, fq=fq))
        conv8.set_tile(tile)
        ref8 = DeviceTensor(n, 14, 14, 256, U8B)
        out8 = DeviceTensor(n, 14, 14, 256, U8B)
        conv8.run(xin, ref8)
        conv8.run_static(xin, out8)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(out8.to_nchw(), ref8.to_nchw())


def test_static_scratch_entry_point_runs_every_other_variant_unchanged(orc):
    """variants without a workspace take the same path through both entry points"""
    import torch
    from dldt_amd import Convolution, DeviceTensor
    rng = np.random.default_rng(71)
    x, w = _case(rng, 2, 128, 12, 96, 3)
    xin = DeviceTensor.from_nchw(x, U8B, halo=1)
    want = orc.convolution(x, w, (1, 1), (1, 1), (1, 1), (1, 1))
    for tile in (0, 4, 18):
        conv = Convolution(w.astype(np.int8), xin, pads_begin=(1, 1), pads_end=(1, 1))
        conv.set_tile(tile)
        out = DeviceTensor(2, 12, 12, 96, I32)
        conv.run_static(xin, out)
        torch.cuda.synchronize()
        np.testing.assert_array_equal(out.to_nchw(), want)


def test_static_scratch_entry_point_refuses_what_does_not_fit():
    from dldt_amd import Convolution, DeviceTensor, HipieError
    rng = np.random.default_rng(72)
    x, w = _case(rng, 20, 64, 28, 320, 3)              # 123 pixel tiles x 3 channel tiles x 4 parts > 256 blocks
    xin = DeviceTensor.from_nchw(x, U8B, halo=1)
    conv = Convolution(w.astype(np.int8), xin, pads_begin=(1, 1), pads_end=(1, 1))
    conv.set_tile(15)
    out = DeviceTensor(20, 28, 28, 320, I32)
    with pytest.raises(HipieError) as e:
        conv.run_static(xin, out)
    assert e.value.status == -6 and "static scratch" in str(e.value)
    conv.run(xin, out)                                  # the allocating entry point takes it
