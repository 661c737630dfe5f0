"""One BERT encoder layer (benchmark configuration 5 at reduced width) composed from the C-ABI operators,
checked segment by segment against the oracle.

The fp32 glue (softmax, LayerNorm, GELU) has tolerance parity only, and a FakeQuantize behind it can
turn a last-ulp difference into a level, so each segment is evaluated by the oracle from the DEVICE's
input tensors of that segment: integer GEMMs, dequantisation, requantisation, residual adds and the
data movement (head slicing by strides, the V transpose) must then be bit-exact, the glue within its
tolerance.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _fq_i8(orc, x, absmax):
    from dldt_amd.bert import sym_i8_range
    il, ih, _ = sym_i8_range(absmax)
    return orc.fake_quantize(x, il, ih, np.float32(-128), np.float32(127), 256).astype(np.int8)


def _linear(orc, xq, layer, name):
    """(acc + b') * scale with the layer's constants: Convert(i32 -> f32), Add, Multiply."""
    acc = orc.matmul(xq.astype(np.int32), layer.wq[name].astype(np.int32), False, True).astype(np.float32)
    return orc.multiply(orc.add(acc, layer.c[name]["bias"]), layer.c[name]["scale"])


def test_encoder_layer_segments_match_the_oracle(orc):
    import torch
    from dldt_amd.bert import EncoderLayer
    B, S, H, NH, FF = 2, 128, 128, 2, 256
    layer = EncoderLayer(hidden=H, heads=NH, ffn=FF, batch=B, seq=S, seed=7)
    rng = np.random.default_rng(70)
    x = rng.normal(0, 1, (B, S, H)).astype(np.float32)
    y = layer.run(torch.from_numpy(x).cuda())
    torch.cuda.synchronize()
    t = {k: v.cpu().numpy() for k, v in layer.t.items()}
    T = B * S
    x2 = x.reshape(T, H)

    # 1. input quantisation, QKV GEMM with per-segment requantisation
    xq = _fq_i8(orc, x2, layer.r["x"])
    np.testing.assert_array_equal(t["xq"], xq)
    f = _linear(orc, xq, layer, "qkv")
    il, ih = layer.c["qkv_fq"]
    qkv = orc.fake_quantize(f, il, ih, np.float32(-128), np.float32(127), 256).astype(np.int8)
    np.testing.assert_array_equal(t["qkv"], qkv)
    assert len(np.unique(qkv)) > 60            # the ranges are exercised, not saturated

    # 2. attention scores per (batch, head): heads are column slices of [T, 3H]
    q = qkv[:, :H].reshape(B, S, NH, 64).transpose(0, 2, 1, 3).astype(np.int32)
    k = qkv[:, H:2 * H].reshape(B, S, NH, 64).transpose(0, 2, 1, 3).astype(np.int32)
    v = qkv[:, 2 * H:].reshape(B, S, NH, 64).transpose(0, 2, 1, 3)
    scores = orc.multiply(orc.matmul(q, k, False, True).astype(np.float32), layer.c["scores_scale"])
    np.testing.assert_array_equal(t["scores"].view(np.uint32), scores.view(np.uint32))
    np.testing.assert_array_equal(t["vt"], v.transpose(0, 1, 3, 2))          # Transpose node

    # 3. softmax (tolerance), then from the device's probabilities: FQ, context GEMM, head merge
    np.testing.assert_allclose(t["p"].reshape(B, NH, S, S), orc.softmax(scores, -1), rtol=2e-6, atol=1e-8)
    pq = _fq_i8(orc, t["p"], layer.r["p"])
    np.testing.assert_array_equal(t["pq"].reshape(pq.shape), pq)
    ctx = orc.multiply(orc.matmul(pq.reshape(B, NH, S, S).astype(np.int32), v.astype(np.int32)).astype(np.float32),
                       layer.c["ctx_scale"])
    ctx = ctx.transpose(0, 2, 1, 3).reshape(T, H)
    np.testing.assert_array_equal(t["ctx"].view(np.uint32), np.ascontiguousarray(ctx).view(np.uint32))

    # 4. output projection with the f32 residual, LayerNorm (tolerance)
    ctxq = _fq_i8(orc, ctx, layer.r["ctx"])
    np.testing.assert_array_equal(t["ctxq"], ctxq)
    attn = orc.add(_linear(orc, ctxq, layer, "o"), x2)
    np.testing.assert_array_equal(t["attn"].view(np.uint32), attn.view(np.uint32))
    g1, b1 = layer.ln[0]
    np.testing.assert_allclose(t["h1"], orc.add(orc.multiply(orc.mvn_last_axis(attn, True, 1e-5, True), g1), b1),
                               rtol=1e-5, atol=4e-6)

    # 5. FFN from the device's h1: FQ, up GEMM, GELU (tolerance), FQ, down GEMM + residual, LayerNorm
    h1q = _fq_i8(orc, t["h1"], layer.r["h1"])
    np.testing.assert_array_equal(t["h1q"], h1q)
    up = _linear(orc, h1q, layer, "up")
    np.testing.assert_array_equal(t["f"].view(np.uint32), up.view(np.uint32))
    np.testing.assert_allclose(t["gelu"], orc.gelu_erf(up), rtol=1e-6, atol=1e-8)
    gq = _fq_i8(orc, t["gelu"], layer.r["g"])
    np.testing.assert_array_equal(t["gq"], gq)
    o = orc.add(_linear(orc, gq, layer, "down"), t["h1"])
    np.testing.assert_array_equal(t["o"].view(np.uint32), o.view(np.uint32))
    g2, b2 = layer.ln[1]
    want_y = orc.add(orc.multiply(orc.mvn_last_axis(o, True, 1e-5, True), g2), b2)
    np.testing.assert_allclose(y.cpu().numpy().reshape(T, H), want_y, rtol=1e-5, atol=4e-6)
