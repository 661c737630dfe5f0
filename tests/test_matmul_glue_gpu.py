"""MatMul on int8 MFMA (constant weights and activation x activation, benchmark configuration 5 shapes) and
the fp32 glue (softmax, MVN/LayerNorm, GELU) through the C ABI vs the oracle."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

F32, I8, I32, U8B = 10, 50, 70, 41


@pytest.mark.parametrize("batch,m,k,n", [(6, 384, 64, 384), (6, 384, 384, 64), (3, 100, 128, 200), (2, 7, 64, 40)])
def test_batched_matmul_i8_exact(orc, batch, m, k, n):
    """Attention scores [S,64]x[64,S] and context [S,S]x[S,64]: exact i32 = reference matmul<int32_t>."""
    import torch
    from dldt_amd import BatchedMatMul
    rng = np.random.default_rng(m + n)
    a = rng.integers(-128, 128, (batch, m, k)).astype(np.int8)
    bt = rng.integers(-128, 128, (batch, n, k)).astype(np.int8)
    want = orc.matmul(a.astype(np.int32), bt.astype(np.int32), False, True)
    got = BatchedMatMul(k, n).run(torch.from_numpy(a).cuda(), torch.from_numpy(bt).cuda()).cpu().numpy()
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("batch,m,k,n,zp", [(6, 384, 384, 64, 0), (3, 100, 128, 200, 0), (2, 7, 64, 40, 17), (5, 130, 192, 128, 255)])
def test_batched_matmul_u8_left_operand(orc, batch, m, k, n, zp):
    """u8 levels (a quantized Softmax output) times an i8 activation: exact i32 sums of (q - zero point) * b, the u8
    operand stored as level - 128 and the row sums of the right operand folded into the accumulators' start; then the
    dequantizing Multiply and the next FakeQuantize in the same kernel"""
    import torch
    from dldt_amd import BatchedMatMul, make_epilogue
    rng = np.random.default_rng(m + n + zp)
    a = rng.integers(0, 256, (batch, m, k)).astype(np.int32)
    bt = rng.integers(-128, 128, (batch, n, k)).astype(np.int8)
    want = orc.matmul(a - zp, bt.astype(np.int32), False, True)
    ad = torch.from_numpy((a - 128).astype(np.int8)).cuda()
    bd = torch.from_numpy(bt).cuda()
    mm = BatchedMatMul(k, n, a_dtype=U8B, a_zero_point=zp)
    np.testing.assert_array_equal(mm.run(ad, bd).cpu().numpy(), want)
    np.testing.assert_array_equal(mm.run(ad, bd).cpu().numpy(), want)        # the workspace of a second call is its own
    s = np.float32(1 / 255) * np.float32(0.03)
    f = orc.multiply(want.astype(np.float32), s)
    hi = np.float32(np.abs(f).max())
    lo = np.float32(-hi * np.float32(128) / np.float32(127))
    lv = orc.fake_quantize(f, lo, hi, np.float32(-128), np.float32(127), 256).astype(np.int8)
    got8 = BatchedMatMul(k, n, make_epilogue(scale=[s], out_dtype=I8, fq=(256, lo, hi, -128.0, 127.0)), a_dtype=U8B,
                         a_zero_point=zp).run(ad, bd)
    np.testing.assert_array_equal(got8.cpu().numpy(), lv)


@pytest.mark.parametrize("batch,m,k,n,za,zb", [(4, 384, 64, 384, None, 0), (3, 100, 128, 200, None, 0), (2, 7, 64, 40, None, 9),
                                               (3, 130, 192, 128, 0, 0), (2, 257, 64, 72, 31, 200), (1, 64, 128, 64, 255, 255)])
def test_batched_matmul_u8_right_operand(orc, batch, m, k, n, za, zb):
    """A u8 right operand (an activation quantized behind a ReLU), against an i8 (za None) or a u8 left operand: exact
    i32 sums of (a - za)(b - zb).  Stored as level - 128, the right operand asks for one correction per output row
    (the sums over K of the left operand's rows), added to the accumulators in front of the epilogue."""
    import torch
    from dldt_amd import BatchedMatMul, make_epilogue
    rng = np.random.default_rng(m + n + zb)
    if za is None:
        a = rng.integers(-128, 128, (batch, m, k)).astype(np.int32)
        a_stored, kw = a.astype(np.int8), {}
        a_real = a
    else:
        a = rng.integers(0, 256, (batch, m, k)).astype(np.int32)
        a_stored, kw = (a - 128).astype(np.int8), dict(a_dtype=U8B, a_zero_point=za)
        a_real = a - za
    bt = rng.integers(0, 256, (batch, n, k)).astype(np.int32)
    want = orc.matmul(a_real, bt - zb, False, True)
    ad = torch.from_numpy(a_stored).cuda()
    bd = torch.from_numpy((bt - 128).astype(np.int8)).cuda()
    mm = BatchedMatMul(k, n, b_dtype=U8B, b_zero_point=zb, **kw)
    np.testing.assert_array_equal(mm.run(ad, bd).cpu().numpy(), want)
    np.testing.assert_array_equal(mm.run(ad, bd).cpu().numpy(), want)
    s = np.float32(1 / 255) * np.float32(0.02)
    f = orc.multiply(want.astype(np.float32), s)
    hi = np.float32(np.abs(f).max())
    lo = np.float32(-hi * np.float32(128) / np.float32(127))
    lv = orc.fake_quantize(f, lo, hi, np.float32(-128), np.float32(127), 256).astype(np.int8)
    got8 = BatchedMatMul(k, n, make_epilogue(scale=[s], out_dtype=I8, fq=(256, lo, hi, -128.0, 127.0)), b_dtype=U8B,
                         b_zero_point=zb, **kw).run(ad, bd)
    np.testing.assert_array_equal(got8.cpu().numpy(), lv)
    gotf = BatchedMatMul(k, n, make_epilogue(scale=[s], out_dtype=F32), b_dtype=U8B, b_zero_point=zb, **kw).run(ad, bd)
    np.testing.assert_array_equal(gotf.cpu().numpy().view(np.uint32), f.view(np.uint32))


def test_batched_matmul_u8_needs_its_workspace_and_a_level_as_zero_point():
    import ctypes
    import torch
    from dldt_amd import BatchedMatMul, HipieError
    from dldt_amd.ops import matmul_strided
    with pytest.raises(HipieError):
        BatchedMatMul(64, 64, a_dtype=U8B, a_zero_point=256)
    with pytest.raises(HipieError):
        BatchedMatMul(64, 64, a_zero_point=3)                      # an i8 operand has none
    with pytest.raises(HipieError):
        BatchedMatMul(64, 64, b_dtype=U8B, b_zero_point=-1)
    with pytest.raises(HipieError):
        BatchedMatMul(64, 64, b_zero_point=3)
    a = torch.zeros((1, 64, 64), dtype=torch.int8, device="cuda")
    out = torch.zeros((1, 64, 64), dtype=torch.int32, device="cuda")
    with pytest.raises(HipieError) as e:
        matmul_strided(BatchedMatMul(64, 64, b_dtype=U8B), a.data_ptr(), 64, 0, a.data_ptr(), 64, 0, out.data_ptr(), 64, 0, 64, 1)
    assert "workspace" in str(e.value)
    mm = BatchedMatMul(64, 64, a_dtype=U8B)
    a = torch.zeros((1, 64, 64), dtype=torch.int8, device="cuda")
    out = torch.zeros((1, 64, 64), dtype=torch.int32, device="cuda")
    with pytest.raises(HipieError) as e:
        matmul_strided(mm, a.data_ptr(), 64, 0, a.data_ptr(), 64, 0, out.data_ptr(), 64, 0, 64, 1)
    assert "workspace" in str(e.value)


def test_batched_matmul_scaled_and_requantized(orc):
    """MatMul' -> Multiply(s_a * s_b) -> f32, and -> FakeQuantize (symmetric i8) as the next MatMul wants it."""
    import torch
    from dldt_amd import BatchedMatMul, make_epilogue
    rng = np.random.default_rng(3)
    batch, m, k, n = 4, 96, 64, 128
    a = rng.integers(-128, 128, (batch, m, k)).astype(np.int8)
    bt = rng.integers(-128, 128, (batch, n, k)).astype(np.int8)
    acc = orc.matmul(a.astype(np.int32), bt.astype(np.int32), False, True).astype(np.float32)
    s = np.float32(0.02) * np.float32(0.03)                 # mat_mul_transformation.cpp:156-174 golden: 0.0006
    want = orc.multiply(acc, s)
    ad, bd = torch.from_numpy(a).cuda(), torch.from_numpy(bt).cuda()
    got = BatchedMatMul(k, n, make_epilogue(scale=[s], out_dtype=F32)).run(ad, bd).cpu().numpy()
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))
    hi = np.float32(np.abs(want).max())
    lo = np.float32(-hi * np.float32(128) / np.float32(127))
    lv = orc.fake_quantize(want, lo, hi, np.float32(-128), np.float32(127), 256).astype(np.int8)
    got8 = BatchedMatMul(k, n, make_epilogue(scale=[s], out_dtype=I8, fq=(256, lo, hi, -128.0, 127.0))).run(ad, bd)
    np.testing.assert_array_equal(got8.cpu().numpy(), lv)


def test_fc_matmul_constant_weights(orc):
    """FC [N,2048] x [2048,1000]^T as the 1x1 convolution path: u8 rows, i8 constant weights."""
    from dldt_amd import Convolution, DeviceTensor
    rng = np.random.default_rng(11)
    x = rng.integers(0, 256, (5, 2048, 1, 1)).astype(np.int32)
    w = rng.integers(-127, 128, (1000, 2048, 1, 1)).astype(np.int32)
    want = orc.matmul(x[:, :, 0, 0], w[:, :, 0, 0], False, True)
    xin = DeviceTensor.from_nchw(x, U8B)
    out = DeviceTensor(5, 1, 1, 1000, I32)
    Convolution(w.astype(np.int8), xin).run(xin, out)
    np.testing.assert_array_equal(out.to_nchw()[:, :, 0, 0], want)


@pytest.mark.parametrize("rows,k,n", [(64, 2048, 1000), (5, 2048, 1000), (70, 1280, 1000), (9, 64, 72), (3, 4096, 136), (1, 192, 64)])
def test_few_pixel_kernel_on_fc_layers(orc, rows, k, n):
    """the variant for 1 x 1 layers with few pixels and many channels (a lane per output channel, K split over the
    four waves of a workgroup, weights packed K-major): raw i32 sums and the bias / scale [/ ReLU] tail to f32 bit for
    bit, pixel counts that are not a multiple of 8, channel counts that are not a multiple of 64, K of one piece per wave
    and of two rounds"""
    from dldt_amd import Convolution, DeviceTensor, HipieError, make_epilogue
    rng = np.random.default_rng(rows * 7 + n)
    x = rng.integers(0, 256, (rows, k, 1, 1)).astype(np.int32)
    w = rng.integers(-127, 128, (n, k, 1, 1)).astype(np.int32)
    acc = orc.matmul(x[:, :, 0, 0], w[:, :, 0, 0], False, True)
    xin = DeviceTensor.from_nchw(x, U8B)
    conv = Convolution(w.astype(np.int8), xin)
    conv.set_tile(23)
    assert conv.get_tile() == 23
    out = DeviceTensor(rows, 1, 1, n, I32)
    conv.run(xin, out)
    np.testing.assert_array_equal(out.to_nchw()[:, :, 0, 0], acc)
    bias = rng.normal(0, 500, n).astype(np.float32)
    scale = rng.uniform(1e-4, 3e-4, n).astype(np.float32)
    for relu in (False, True):
        want = orc.multiply(orc.add(acc.astype(np.float32), bias), scale)
        if relu:
            want = orc.relu(want)
        conv = Convolution(w.astype(np.int8), xin, epilogue=make_epilogue(bias=bias, scale=scale, activation="relu" if relu else None,
                                                                         out_dtype=F32))
        outs = {}
        for tile in (0, 23):
            conv.set_tile(tile)
            o = DeviceTensor(rows, 1, 1, n, F32)
            conv.run(xin, o)
            outs[tile] = o.to_nchw()[:, :, 0, 0]
        np.testing.assert_array_equal(outs[23].view(np.uint32), want.view(np.uint32))
        np.testing.assert_array_equal(outs[0].view(np.uint32), want.view(np.uint32))
    # a requantizing tail is not this kernel's: refused, the layer keeps its variant
    fq = (256, 0.0, np.float32(4.0), 0.0, 255.0)
    conv = Convolution(w.astype(np.int8), xin, epilogue=make_epilogue(bias=bias, scale=scale, out_dtype=U8B, fq=fq))
    with pytest.raises(HipieError):
        conv.set_tile(23)


def test_softmax_mvn_gelu_tolerance(orc):
    import torch
    from dldt_amd import gelu, mvn, softmax
    rng = np.random.default_rng(13)
    x = (rng.standard_normal((2, 12, 48, 384)) * 3).astype(np.float32)
    xd = torch.from_numpy(x).cuda()
    np.testing.assert_allclose(softmax(xd).cpu().numpy(), orc.softmax(x, -1), rtol=2e-6, atol=1e-8)
    h = (rng.standard_normal((96, 768)) * 2 + 0.3).astype(np.float32)
    hd = torch.from_numpy(h).cuda()
    for inside in (True, False):
        np.testing.assert_allclose(mvn(hd, True, 1e-5, inside).cpu().numpy(),
                                   orc.mvn_last_axis(h, True, 1e-5, inside), rtol=1e-5, atol=2e-6)
    gamma = rng.uniform(0.5, 1.5, 768).astype(np.float32)
    beta = rng.normal(0, 0.1, 768).astype(np.float32)
    want = orc.add(orc.multiply(orc.mvn_last_axis(h, True, 1e-5, True), gamma), beta)
    got = mvn(hd, True, 1e-5, True, torch.from_numpy(gamma).cuda(), torch.from_numpy(beta).cuda()).cpu().numpy()
    np.testing.assert_allclose(got, want, rtol=1e-5, atol=2e-6)
    f = (rng.standard_normal((64, 3072)) * 2).astype(np.float32)
    np.testing.assert_allclose(gelu(torch.from_numpy(f).cuda()).cpu().numpy(), orc.gelu_erf(f), rtol=1e-6, atol=1e-8)


@pytest.mark.parametrize("shape,addend", [((2, 3, 40, 64), (2, 1, 1, 64)), ((2, 3, 40, 64), (1, 3, 40, 1)), ((2, 3, 40, 64), (2, 3, 40, 64)),
                                          ((5, 33, 7), (1, 33, 1)), ((6, 10), (6, 1)), ((77,), (77,)), ((4, 2, 9, 5), (1, 1, 1, 1))])
def test_add_with_a_broadcast_addend(orc, shape, addend):
    """reference::add with numpy broadcasting: bit-exact, also in place; an addend that does not broadcast is refused"""
    import torch
    from dldt_amd import HipieError
    from dldt_amd.ops import add_broadcast
    rng = np.random.default_rng(len(shape) * 100 + sum(addend))
    x = (rng.standard_normal(shape) * 5).astype(np.float32)
    m = (rng.standard_normal(addend) * 5).astype(np.float32)
    want = orc.add(x, m)
    xd, md = torch.from_numpy(x).cuda(), torch.from_numpy(m).cuda()
    np.testing.assert_array_equal(add_broadcast(xd, md).cpu().numpy().view(np.uint32), want.view(np.uint32))
    add_broadcast(xd, md, out=xd)
    np.testing.assert_array_equal(xd.cpu().numpy().view(np.uint32), want.view(np.uint32))
    if len(shape) > 1 and shape[-1] > 2:
        with pytest.raises(HipieError) as e:
            add_broadcast(xd, torch.zeros(shape[:-1] + (2,), device="cuda"))
        assert e.value.status == -4


@pytest.mark.parametrize("axis", [4, 64, 100, 252, 384, 390, 768, 1500, 3072, 4100])
def test_glue_row_lengths(orc, axis):
    """rows held in registers (multiples of 4 up to 4096, partial last chunk) and the three-pass fallback"""
    import torch
    from dldt_amd import mvn, softmax
    rng = np.random.default_rng(axis)
    x = (rng.standard_normal((37, axis)) * 3).astype(np.float32)
    xd = torch.from_numpy(x).cuda()
    np.testing.assert_allclose(softmax(xd).cpu().numpy(), orc.softmax(x, -1), rtol=3e-6, atol=1e-8)
    tol = dict(rtol=2e-5, atol=4e-6)
    np.testing.assert_allclose(mvn(xd).cpu().numpy(), orc.mvn_last_axis(x, True, 1e-5, True), **tol)
    np.testing.assert_allclose(mvn(xd, False).cpu().numpy(), orc.mvn_last_axis(x, False, 1e-5, True), **tol)


def _fq_i8(orc, v, il, ih):
    return orc.fake_quantize(v, np.float32(il), np.float32(ih), np.float32(-128), np.float32(127), 256).astype(np.int8)


@pytest.mark.parametrize("axis", [384, 100, 390])
def test_glue_with_fused_requantisation(orc, axis):
    """The fused i8 output equals the reference FakeQuantize of the kernel's own f32 result bit for bit,
    and the f32 result does not depend on whether the quantized output is asked for."""
    import torch
    from dldt_amd import gelu, mvn, softmax
    rng = np.random.default_rng(5 + axis)
    x = (rng.standard_normal((61, axis)) * 2).astype(np.float32)
    xd = torch.from_numpy(x).cuda()
    gamma = torch.from_numpy(rng.uniform(0.5, 1.5, axis).astype(np.float32)).cuda()
    beta = torch.from_numpy(rng.normal(0, 0.1, axis).astype(np.float32)).cuda()
    il, ih = np.float32(-128) * np.float32(1.0 / 127), np.float32(1.0)
    cases = [
        ("softmax", lambda **k: softmax(xd, **k), (il * np.float32(0.2), ih * np.float32(0.2))),
        ("mvn", lambda **k: mvn(xd, True, 1e-5, True, gamma, beta, **k), (il * 2, ih * 2)),
        ("gelu", lambda **k: gelu(xd, **k), (il * 3, ih * 3)),
    ]
    for name, fn, (lo, hi) in cases:
        plain = fn().cpu().numpy()
        y, q = fn(requant=(lo, hi, -128, 256))
        np.testing.assert_array_equal(y.cpu().numpy().view(np.uint32), plain.view(np.uint32), err_msg=name)
        want = _fq_i8(orc, plain, lo, hi)
        np.testing.assert_array_equal(q.cpu().numpy(), want, err_msg=name)
        assert len(np.unique(want)) > 40, name
        if axis % 4 == 0:                                   # f32 output left out: register-resident rows only
            q_only = fn(requant=(lo, hi, -128, 256), keep_f32=False)
            np.testing.assert_array_equal(q_only.cpu().numpy(), want, err_msg=name)


def test_glue_requantisation_rejects_non_integer_levels():
    import torch
    from dldt_amd import HipieError, gelu
    x = torch.zeros((4, 64), device="cuda")
    with pytest.raises(HipieError):
        gelu(x, requant=(-1.0, 1.0, -0.5, 256))
    with pytest.raises(HipieError):
        gelu(x, requant=(1.0, -1.0, -128, 256))


@pytest.mark.parametrize("B,NH,S", [(2, 3, 384), (1, 2, 96), (2, 1, 160), (1, 1, 32),
                                    (4, 4, 160), (2, 8, 64)])      # 16 batch elements: the grid that groups neighbouring heads per XCD
def test_fused_attention(orc, B, NH, S):
    """scores bit-exact, Softmax within tolerance, and from the kernel's own probabilities the
    requantisation, the context product and its dequantisation (and requantisation) bit-exact; the
    kernel without the inspection outputs gives the same bytes.  q, k, v are head slices of one
    [tokens, 3 * hidden] tensor, as a fused QKV projection leaves them."""
    import torch
    from dldt_amd import attention
    rng = np.random.default_rng(S + NH)
    H = NH * 64
    qkv = rng.integers(-128, 128, (B, S, 3, NH, 64), dtype=np.int8)
    qkv[:, :, 0] = np.clip(rng.normal(0, 20, (B, S, NH, 64)), -128, 127).astype(np.int8)
    t = torch.from_numpy(qkv).cuda()
    q, k, v = (t[:, :, i].permute(0, 2, 1, 3) for i in range(3))           # [B, NH, S, 64] views, row pitch 3 H
    assert q.stride(2) == 3 * H
    s1, s2 = np.float32(0.0007), np.float32(0.02 / 127)
    il, ih = np.float32(-128.0 / 127), np.float32(1.0)
    ctx, scores, probs = attention(q, k, v, s1, s2, (il, ih, -128, 256), dump=True)
    qn, kn, vn = (np.ascontiguousarray(x.cpu().numpy()).astype(np.int32) for x in (q, k, v))
    want_scores = orc.multiply(orc.matmul(qn, kn, False, True).astype(np.float32), s1)
    np.testing.assert_array_equal(scores.cpu().numpy().view(np.uint32), want_scores.view(np.uint32))
    p = probs.cpu().numpy()
    np.testing.assert_allclose(p, orc.softmax(want_scores, -1), rtol=3e-6, atol=1e-8)
    pq = orc.fake_quantize(p, il, ih, np.float32(-128), np.float32(127), 256).astype(np.int32)
    assert len(np.unique(pq)) > 20
    want_ctx = orc.multiply(orc.matmul(pq, vn).astype(np.float32), s2)
    np.testing.assert_array_equal(ctx.cpu().numpy().view(np.uint32), want_ctx.view(np.uint32))
    plain = attention(q, k, v, s1, s2, (il, ih, -128, 256))
    assert torch.equal(plain, ctx)
    # requantised output
    ol, oh = np.float32(-128) * np.float32(0.004), np.float32(127) * np.float32(0.004)
    cq = attention(q, k, v, s1, s2, (il, ih, -128, 256), out_fq=(ol, oh, -128, 256))
    want_q = orc.fake_quantize(want_ctx, ol, oh, np.float32(-128), np.float32(127), 256).astype(np.int8)
    np.testing.assert_array_equal(cq.cpu().numpy(), want_q)
    assert len(np.unique(want_q)) > 40


def test_fused_attention_rejects_unsupported_shapes():
    import torch
    from dldt_amd import HipieError, attention
    for shape in [(1, 1, 48, 64), (1, 1, 416, 64), (1, 1, 64, 32)]:
        x = torch.zeros(shape, dtype=torch.int8, device="cuda")
        with pytest.raises(HipieError) as e:
            attention(x, x, x, 1.0, 1.0, (-1.0, 1.0, -128, 256))
        assert e.value.status == -2


def test_fused_attention_with_mask(orc):
    """additive mask row per sequence, shared by its heads: added to the scaled scores in front of the Softmax"""
    import torch
    from dldt_amd.ops import Attention
    rng = np.random.default_rng(77)
    B, NH, S = 3, 2, 160
    t = torch.from_numpy(rng.integers(-60, 61, (B, S, 3, NH, 64), dtype=np.int8)).cuda()
    q, k, v = (t[:, :, i].permute(0, 2, 1, 3) for i in range(3))
    mask = np.zeros((B, S), np.float32)
    mask[0, 100:] = -10000.0
    mask[2, 7:] = -10000.0
    mask[1] = rng.normal(0, 1, S).astype(np.float32)                       # any additive row, not only 0 / -10000
    s1, s2 = np.float32(0.002), np.float32(0.01)
    il, ih = np.float32(-128.0 / 127), np.float32(1.0)
    att = Attention(S, 64, s1, s2, (il, ih, -128, 256))
    ctx, scores, probs = att.run(q, k, v, dump=True, mask=torch.from_numpy(mask).cuda())
    qn, kn, vn = (np.ascontiguousarray(x.cpu().numpy()).astype(np.int32) for x in (q, k, v))
    want_scores = orc.add(orc.multiply(orc.matmul(qn, kn, False, True).astype(np.float32), s1), mask[:, None, None, :])
    np.testing.assert_array_equal(scores.cpu().numpy().view(np.uint32), want_scores.view(np.uint32))
    p = probs.cpu().numpy()
    np.testing.assert_allclose(p, orc.softmax(want_scores, -1), rtol=3e-6, atol=1e-8)
    assert p[0, :, :, 100:].max() == 0.0 and p[2, :, :, 7:].max() == 0.0
    pq = orc.fake_quantize(p, il, ih, np.float32(-128), np.float32(127), 256).astype(np.int32)
    want_ctx = orc.multiply(orc.matmul(pq, vn).astype(np.float32), s2)
    np.testing.assert_array_equal(ctx.cpu().numpy().view(np.uint32), want_ctx.view(np.uint32))
    assert torch.equal(att.run(q, k, v, mask=torch.from_numpy(mask).cuda()), ctx)


@pytest.mark.parametrize("S,masked", [(128, False), (384, False), (160, True)])
def test_fused_attention_with_u8_probabilities(orc, S, masked):
    """the Softmax output quantized to u8 levels 0..255: stored as level - 128 for the signed matrix instruction, the
    sums of V over the keys (times 128) start the accumulators of the context product"""
    import torch
    from dldt_amd.ops import Attention
    rng = np.random.default_rng(S)
    B, NH = 2, 3
    t = torch.from_numpy(rng.integers(-70, 71, (B, S, 3, NH, 64), dtype=np.int8)).cuda()
    q, k, v = (t[:, :, i].permute(0, 2, 1, 3) for i in range(3))
    s1, s2 = np.float32(0.002), np.float32(0.01) / np.float32(255)
    il, ih = np.float32(0.0), np.float32(1.0)
    mask = None
    if masked:
        mask = np.zeros((B, S), np.float32)
        mask[1, 90:] = -10000.0
    att = Attention(S, 64, s1, s2, (il, ih, -128, 256), prob_dtype=U8B)
    md = torch.from_numpy(mask).cuda() if masked else None
    ctx, scores, probs = att.run(q, k, v, dump=True, mask=md)
    qn, kn, vn = (np.ascontiguousarray(x.cpu().numpy()).astype(np.int32) for x in (q, k, v))
    want_scores = orc.multiply(orc.matmul(qn, kn, False, True).astype(np.float32), s1)
    if masked:
        want_scores = orc.add(want_scores, mask[:, None, None, :])
    np.testing.assert_array_equal(scores.cpu().numpy().view(np.uint32), want_scores.view(np.uint32))
    p = probs.cpu().numpy()
    np.testing.assert_allclose(p, orc.softmax(want_scores, -1), rtol=3e-6, atol=1e-8)
    pq = orc.fake_quantize(p, il, ih, np.float32(0), np.float32(255), 256).astype(np.int32)    # from the device's f32 probabilities
    assert pq.max() > 128 or S > 128
    want_ctx = orc.multiply(orc.matmul(pq, vn).astype(np.float32), s2)
    np.testing.assert_array_equal(ctx.cpu().numpy().view(np.uint32), want_ctx.view(np.uint32))
    assert torch.equal(att.run(q, k, v, mask=md), ctx)


def test_nested_batches_inside_a_packed_tensor():
    """hipie_matmul_run_nested / hipie_transpose_bytes_nested address (sequence, head) batches inside one
    [tokens, 3 * hidden] tensor by pitch, inner and outer strides (the attention operands of an encoder without
    copying the heads out): q k^T per head against numpy's integer product, and V transposed per head"""
    import torch
    from dldt_amd import BatchedMatMul, make_epilogue
    from dldt_amd.ops import matmul_strided, transpose_bytes
    from dldt_amd.tensor import I32
    rng = np.random.default_rng(77)
    B, S, NH, D = 2, 96, 3, 64
    H = NH * D
    qkv = rng.integers(-128, 128, (B * S, 3 * H)).astype(np.int8)
    t = torch.from_numpy(qkv).cuda()
    scores = torch.zeros((B, NH, S, S), dtype=torch.int32, device="cuda")
    mm = BatchedMatMul(D, S, make_epilogue(out_dtype=I32))
    base = t.data_ptr()
    # head h of sequence b: rows b * S .., columns h * D .. (q) and H + h * D .. (k)
    matmul_strided(mm, base, 3 * H, D, base + H, 3 * H, D, scores.data_ptr(), S, S * S, S, NH,
                   batch_outer=B, outer_a=S * 3 * H, outer_b=S * 3 * H, outer_o=NH * S * S)
    x = qkv.reshape(B, S, 3, NH, D).astype(np.int64)
    want = np.einsum("bshd,bthd->bhst", x[:, :, 0], x[:, :, 1])
    np.testing.assert_array_equal(scores.cpu().numpy(), want)
    vt = torch.zeros((B, NH, D, S), dtype=torch.int8, device="cuda")
    transpose_bytes(base + 2 * H, 3 * H, D, vt.data_ptr(), S, D * S, S, D, NH, batch_outer=B,
                    outer_src=S * 3 * H, outer_dst=NH * D * S)
    np.testing.assert_array_equal(vt.cpu().numpy(), qkv.reshape(B, S, 3, NH, D)[:, :, 2].transpose(0, 2, 3, 1))
