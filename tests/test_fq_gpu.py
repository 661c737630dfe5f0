"""FakeQuantize on the GPU through the C ABI vs the oracle (bit-exact)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _per_channel_case(rng, N, C, H, W):
    """benchmark configuration 2 recipe: x ~ N(mu_c, 1), bounds = channel mean -+ 3 sigma."""
    mu = rng.uniform(-0.5, 0.5, C).astype(np.float32)
    x = (rng.standard_normal((N, C, H, W), dtype=np.float32) + mu.reshape(1, C, 1, 1)).astype(np.float32)
    m = x.mean(axis=(0, 2, 3), dtype=np.float64)
    s = x.std(axis=(0, 2, 3), dtype=np.float64)
    return x, (m - 3 * s).astype(np.float32), (m + 3 * s).astype(np.float32)


@pytest.mark.parametrize("shape", [(2, 16, 14, 14), (3, 5, 7, 9), (1, 64, 56, 56), (2, 256, 8, 8), (2, 100, 20, 13), (2, 130, 30, 30),
                                   (1, 72, 4, 257), (1, 300, 6, 10), (2, 512, 12, 12), (1, 128, 1, 4)])
def test_fq_levels_bit_exact(orc, shape):
    import torch
    from dldt_amd import FakeQuantize
    rng = np.random.default_rng(20211)
    x, il, ih = _per_channel_case(rng, *shape)
    C = shape[1]
    bshape = (1, C, 1, 1)
    want = orc.fake_quantize(x, il.reshape(bshape), ih.reshape(bshape), np.float32(0), np.float32(255), 256)
    fq = FakeQuantize(C, 256, il, ih, 0.0, 255.0)
    xd = torch.from_numpy(x).cuda()
    got = fq.run_q8(xd, "u8", "nchw").cpu().numpy()
    np.testing.assert_array_equal(got, want.astype(np.uint8))
    gotf = fq.run_f32(xd).cpu().numpy()
    np.testing.assert_array_equal(gotf.view(np.uint32), want.view(np.uint32))
    # engine-internal storage: NHWC, level - 128, channels padded with level 0
    cs = -(-C // 16) * 16
    nhwc = fq.run_q8(xd, "u8b", "nhwc", cs).cpu().numpy()
    lv = (nhwc.astype(np.int16) + 128).astype(np.uint8)
    np.testing.assert_array_equal(lv[..., :C], want.astype(np.uint8).transpose(0, 2, 3, 1))
    assert np.all(lv[..., C:] == 0)


def test_fq_tie_dense_and_saturation(orc):
    import torch
    from dldt_amd import FakeQuantize
    rng = np.random.default_rng(5)
    C = 32
    il = rng.uniform(-3, -1, C).astype(np.float32)
    ih = rng.uniform(1, 3, C).astype(np.float32)
    k = np.arange(255, dtype=np.float32) + np.float32(0.5)
    mid = (il.reshape(C, 1) + (ih - il).reshape(C, 1) * (k / np.float32(255))).astype(np.float32)
    x = np.concatenate([mid, np.nextafter(mid, np.float32(9)), np.nextafter(mid, np.float32(-9)),
                        np.tile(il.reshape(C, 1), (1, 3)), np.tile(ih.reshape(C, 1), (1, 3)),
                        np.full((C, 4), 1e9, np.float32), np.full((C, 4), -1e9, np.float32)], axis=1)
    x = np.ascontiguousarray(x.reshape(1, C, 1, -1)[..., :776])  # HW % 4 == 0
    want = orc.fake_quantize(x, il.reshape(1, C, 1, 1), ih.reshape(1, C, 1, 1), np.float32(0), np.float32(255), 256)
    fq = FakeQuantize(C, 256, il, ih, 0.0, 255.0)
    got = fq.run_q8(torch.from_numpy(x).cuda(), "u8", "nchw").cpu().numpy()
    np.testing.assert_array_equal(got, want.astype(np.uint8))


@pytest.mark.parametrize("levels,ol,oh", [(4, 2.0, 16.0), (5, 2.0, 16.0), (255, -1.27, 1.27), (16, 0.0, 1.5)])
def test_fq_f32_general_output_ranges(orc, levels, ol, oh):
    import torch
    from dldt_amd import FakeQuantize
    rng = np.random.default_rng(levels)
    x = rng.uniform(-5, 30, (2, 3, 5, 6)).astype(np.float32)
    il, ih = np.float32(0.0 if levels < 16 else -1.27), np.float32(23.0 if levels < 16 else 1.27)
    want = orc.fake_quantize(x, il, ih, np.float32(ol), np.float32(oh), levels)
    fq = FakeQuantize(3, levels, il, ih, ol, oh)
    got = fq.run_f32(torch.from_numpy(x).cuda()).cpu().numpy()
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))


def test_fq_i8_signed_levels(orc):
    import torch
    from dldt_amd import FakeQuantize
    rng = np.random.default_rng(9)
    x = rng.normal(0, 1, (2, 8, 6, 6)).astype(np.float32)
    want = orc.fake_quantize(x, np.float32(-1.28), np.float32(1.27), np.float32(-128), np.float32(127), 256)
    fq = FakeQuantize(8, 256, -1.28, 1.27, -128.0, 127.0)
    got = fq.run_q8(torch.from_numpy(x).cuda(), "i8", "nchw").cpu().numpy()
    np.testing.assert_array_equal(got, want.astype(np.int8))


def test_fq_empty_input():
    import torch
    from dldt_amd import FakeQuantize
    fq = FakeQuantize(4, 256, 0.0, 1.0, 0.0, 255.0)
    y = fq.run_q8(torch.empty((0, 4, 3, 3), device="cuda"), "u8", "nchw")
    assert y.numel() == 0


def test_fq_full_size_properties(orc):
    """benchmark configuration 2 at full size [32,256,56,56]: a seeded sample of planes is compared with
    the oracle; the whole tensor is checked through size-independent properties."""
    import torch
    from dldt_amd import FakeQuantize
    g = torch.Generator(device="cuda").manual_seed(20211)
    N, C, H, W = 32, 256, 56, 56
    mu = (torch.rand(C, generator=g, device="cuda") - 0.5)
    x = torch.randn((N, C, H, W), generator=g, device="cuda") + mu.view(1, C, 1, 1)
    m, s = x.mean(dim=(0, 2, 3)), x.std(dim=(0, 2, 3))
    il, ih = (m - 3 * s).cpu().numpy(), (m + 3 * s).cpu().numpy()
    fq = FakeQuantize(C, 256, il, ih, 0.0, 255.0)
    q = fq.run_q8(x, "u8", "nchw")
    # property: re-quantising the dequantised levels is the identity (idempotence on level grid)
    # property: monotone in x per channel; saturation counts match the 3-sigma tails
    assert q.dtype == torch.uint8 and q.shape == x.shape
    lo_frac = (q == 0).float().mean().item()
    assert 0.0005 < lo_frac < 0.004       # P(x <= mu - 3 sigma) ~ 0.00135 (+ first half-level)
    order = torch.argsort(x[0, 7].flatten())
    assert torch.all(torch.diff(q[0, 7].flatten()[order].int()) >= 0)
    for n, c in ((0, 0), (31, 255), (13, 100)):
        want = orc.fake_quantize(x[n, c].cpu().numpy().reshape(1, 1, H, W), il[c], ih[c],
                                 np.float32(0), np.float32(255), 256)
        np.testing.assert_array_equal(q[n, c].cpu().numpy(), want[0, 0].astype(np.uint8))


def test_two_operation_division_constants_match_ieee_division():
    """fma(x, zh, x * zl) == x / d for the verified constants: spot-check 2 * 10^5 random x per divisor
    against IEEE f32 division on the host (the library itself checks all 2^23 significands)."""
    import ctypes
    from dldt_amd._lib import lib, check
    rng = np.random.default_rng(11)
    d = np.concatenate([rng.uniform(0.01, 3e5, 61).astype(np.float32),
                        np.array([1.0, 255.0, 2.55], np.float32)])
    zh, zl = np.zeros_like(d), np.zeros_like(d)
    ok = ctypes.c_int(0)
    fp = ctypes.POINTER(ctypes.c_float)
    check(lib().hipie_fq_div2_constants(0, d.ctypes.data_as(fp), ctypes.c_int64(d.size), zh.ctypes.data_as(fp),
                                        zl.ctypes.data_as(fp), ctypes.byref(ok)))
    assert ok.value == 1
    assert np.finfo(np.longdouble).nmant >= 63
    x = np.concatenate([rng.uniform(0, 1, 100000), rng.uniform(0, 4e5, 100000)]).astype(np.float32)
    for i in range(d.size):
        lo = x * zl[i]                                                   # one f32 rounding
        # the fma: exact product and a sum rounded once (64-bit significands make a double rounding negligible)
        fast = (x.astype(np.longdouble) * np.longdouble(zh[i]) + lo.astype(np.longdouble)).astype(np.float32)
        np.testing.assert_array_equal(fast, x / d[i])


def test_two_operation_division_reports_unmatched_divisor():
    """A divisor for which no constant pair within the searched neighbourhood reproduces division for
    every significand: the library must say so (the epilogue then keeps the slower exact sequence)."""
    import ctypes
    from dldt_amd._lib import lib, check
    d = np.array([float.fromhex("0x1.e447fep+17")], np.float32)
    zh, zl = np.zeros_like(d), np.zeros_like(d)
    ok = ctypes.c_int(1)
    fp = ctypes.POINTER(ctypes.c_float)
    check(lib().hipie_fq_div2_constants(0, d.ctypes.data_as(fp), ctypes.c_int64(1), zh.ctypes.data_as(fp),
                                        zl.ctypes.data_as(fp), ctypes.byref(ok)))
    assert ok.value == 0
