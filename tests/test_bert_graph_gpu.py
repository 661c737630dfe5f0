"""BERT-style encoder stack (benchmark configuration 5 at reduced width) as a post-LPT graph through the
planner: MatMul against constant weights and between activations, Reshape / Transpose as views,
Softmax, LayerNorm, Gelu, per-tensor FakeQuantize.

The fp32 glue has tolerance parity only and a FakeQuantize behind it can turn a last-ulp difference
into another level, so the oracle interpreter continues from the DEVICE's value behind every glue op:
all integer GEMMs, dequantisations, requantisations, residual adds and data movement must then be
bit-exact, and each glue op is compared with what the oracle makes of the same inputs."""
import numpy as np
import pytest

from interp import evaluate

pytestmark = pytest.mark.gpu

EXACT = ("xq", "q", "k", "v", "scores", "pq", "ctx", "ctxq", "attn", "h1q", "up", "gq", "down")
GLUE_TOL = dict(p=dict(rtol=2e-6, atol=1e-8), h1=dict(rtol=1e-5, atol=4e-6), gelu=dict(rtol=1e-6, atol=1e-8),
                y=dict(rtol=1e-5, atol=4e-6))


def _check_stack(orc, monkeypatch, layers, hidden, heads, ffn, batch, seq, fuse_attention=True, merge_linear=True,
                 unsigned_probs=False):
    from dldt_amd import builders
    monkeypatch.setenv("HIPIE_FUSE_ATTENTION", "1" if fuse_attention else "0")
    monkeypatch.setenv("HIPIE_MERGE_LINEAR", "1" if merge_linear else "0")
    gemms = 4 if merge_linear else 6                         # Q, K, V projections as one GEMM or three
    # first with every f32 value behind a tolerance-only op kept in the arena (segment-wise check) ...
    monkeypatch.setenv("HIPIE_KEEP_F32", "1")
    # ranges for the reduced width: about 30 levels per standard deviation, so the tails saturate
    g, meta = builders.bert_encoder(layers=layers, hidden=hidden, heads=heads, ffn=ffn, batch=batch, seq=seq, seed=7,
                                    ranges=dict(q=0.12, k=0.9, v=0.9, ctx=0.6), unsigned_probs=unsigned_probs)
    x = np.random.default_rng(70).normal(0, 1, (batch, seq, hidden)).astype(np.float32)
    plan = g.compile()
    types = [s["type"] for s in plan.steps]
    if fuse_attention:      # the probabilities stay in registers between the two products
        assert types.count("MatMul") == gemms * layers and types.count("Attention") == layers
        assert "Transpose" not in types and "Softmax+FakeQuantize" not in types
    else:
        assert types.count("MatMul") == (gemms + 2) * layers and types.count("Transpose") == layers
        assert types.count("Softmax+FakeQuantize") == layers
    assert types.count("Gelu+FakeQuantize") == layers
    exact = [n for n in EXACT if not (fuse_attention and n == "pq")]
    req = plan.create_request()
    (y,) = req.infer(x)
    device = {n: req.matrix(n) for n in meta["glue"]}
    keep = [n for L in meta["layers"] for n in L.values()]
    want, kept = evaluate(orc, g.nodes, {"hidden_states": x}, keep=keep, override=device)
    for li, L in enumerate(meta["layers"]):
        for name in exact:
            w = kept[L[name]]
            have = req.matrix(L[name]).reshape(w.shape)
            if w.dtype == np.float32:
                np.testing.assert_array_equal(have.view(np.uint32), w.view(np.uint32), err_msg="layer %d %s" % (li, name))
            else:
                np.testing.assert_array_equal(have.view(np.int8), w.astype(np.int8), err_msg="layer %d %s" % (li, name))
        for name, tol in GLUE_TOL.items():
            w = kept[("oracle", L[name])]
            np.testing.assert_allclose(device[L[name]].reshape(w.shape), w, err_msg="layer %d %s" % (li, name), **tol)
        q = kept[L["q"]]
        assert len(np.unique(q)) > 60                      # the ranges are exercised, not saturated
    np.testing.assert_array_equal(y.view(np.uint32), want["out"].view(np.uint32))
    # ... then as it runs by default: results that only a fused FakeQuantize reads are not stored, the
    # same kernels compute the same bits
    monkeypatch.delenv("HIPIE_KEEP_F32")
    plan2 = g.compile()
    assert len(plan2.steps) < len(plan.steps)
    req2 = plan2.create_request()
    (y2,) = req2.infer(x)
    np.testing.assert_array_equal(y2.view(np.uint32), y.view(np.uint32))
    for li, L in enumerate(meta["layers"]):
        stored = ("q", "k", "v", "ctxq", "attn", "h1q", "gq", "down") + (() if fuse_attention else ("scores", "pq"))
        for name in stored:
            np.testing.assert_array_equal(req2.matrix(L[name]), req.matrix(L[name]), err_msg="layer %d %s" % (li, name))
        for name in ("p", "ctx", "up", "gelu") + (("scores", "pq") if fuse_attention else ()):
            with pytest.raises(Exception):
                req2.matrix(L[name])
    return plan2, req2, x, y


def test_encoder_stack_matches_the_oracle(orc, monkeypatch):
    plan, req, x, y = _check_stack(orc, monkeypatch, layers=2, hidden=128, heads=2, ffn=256, batch=2, seq=128)
    # device-resident path gives the same bytes
    import torch
    ins, outs = req.device_buffers()
    ins[0].copy_(torch.from_numpy(x))
    req.infer_device(ins, outs)
    np.testing.assert_array_equal(outs[0].cpu().numpy(), y)


def test_encoder_stack_other_head_count_and_ragged_rows(orc, monkeypatch):
    """three heads, a sequence length that is not a multiple of the 128-row tiles"""
    _check_stack(orc, monkeypatch, layers=1, hidden=192, heads=3, ffn=320, batch=3, seq=64)


def test_encoder_stack_with_separate_attention_kernels(orc, monkeypatch):
    """the same graph with the attention core planned as MatMul, Softmax + FakeQuantize, Transpose, MatMul"""
    _check_stack(orc, monkeypatch, layers=2, hidden=128, heads=2, ffn=256, batch=2, seq=128, fuse_attention=False)
    _check_stack(orc, monkeypatch, layers=1, hidden=192, heads=3, ffn=320, batch=3, seq=64, fuse_attention=False,
                 merge_linear=False)


def test_encoder_stack_with_u8_probabilities(orc, monkeypatch):
    """the Softmax output quantized to u8 levels 0..255 (what a calibration tool gives a non-negative tensor): the
    context product takes a u8 left operand, with the sums over the keys of V's columns as accumulator corrections -
    in the fused attention kernel and as separate steps"""
    _check_stack(orc, monkeypatch, layers=2, hidden=128, heads=2, ffn=256, batch=2, seq=128, unsigned_probs=True)
    _check_stack(orc, monkeypatch, layers=1, hidden=192, heads=3, ffn=320, batch=3, seq=64, unsigned_probs=True,
                 merge_linear=False)
    _check_stack(orc, monkeypatch, layers=1, hidden=128, heads=2, ffn=256, batch=2, seq=128, unsigned_probs=True,
                 fuse_attention=False)
    _check_stack(orc, monkeypatch, layers=1, hidden=192, heads=3, ffn=320, batch=3, seq=64, unsigned_probs=True,
                 fuse_attention=False)


def test_encoder_stack_with_one_gemm_per_matmul(orc, monkeypatch):
    _check_stack(orc, monkeypatch, layers=1, hidden=128, heads=2, ffn=256, batch=2, seq=128, merge_linear=False)


def test_unsupported_transformer_nodes_are_reported():
    from dldt_amd import HipieError
    from dldt_amd.graph import Graph
    g = Graph()
    x = g.parameter("x", (2, 64, 64))
    g.result(g.softmax(x, 1), "y")                         # not over the last axis
    with pytest.raises(HipieError) as e:
        g.compile()
    assert e.value.status == -2 and "Softmax" in str(e.value)


def test_encoder_with_embedding_front_end(orc, monkeypatch):
    """token ids -> Gather(word table) + position table + token-type row -> LayerNorm -> one encoder layer;
    ids include negative values (counted from the end of the table, gather.hpp:58-59)"""
    from dldt_amd import builders
    monkeypatch.setenv("HIPIE_KEEP_F32", "1")
    B, S, H, V = 2, 64, 128, 500
    g, meta = builders.bert_encoder(layers=1, hidden=H, heads=2, ffn=256, batch=B, seq=S, seed=9, vocab=V,
                                    ranges=dict(q=0.12, k=0.9, v=0.9, ctx=0.6))
    ids = np.random.default_rng(3).integers(-7, V, (B, S)).astype(np.int32)
    assert (ids < 0).any()
    plan = g.compile()
    assert [s["type"] for s in plan.steps[:2]] == ["Gather", "MVN+FakeQuantize"]
    assert plan.inputs[0]["name"] == "input_ids" and plan.inputs[0]["shape"] == (B, S)
    req = plan.create_request()
    (y,) = req.infer(ids)
    device = {n: req.matrix(n) for n in meta["glue"]}
    L = meta["layers"][0]
    keep = [meta["embeddings"]] + [L[k] for k in ("xq", "q", "ctx", "down")]
    want, kept = evaluate(orc, g.nodes, {"input_ids": ids}, keep=keep, override=device)
    emb = kept[meta["embeddings"]]
    np.testing.assert_array_equal(req.matrix(meta["embeddings"]).reshape(emb.shape).view(np.uint32), emb.view(np.uint32))
    w = kept[("oracle", meta["embedding_norm"])]
    np.testing.assert_allclose(device[meta["embedding_norm"]].reshape(w.shape), w, rtol=1e-5, atol=4e-6)
    for k in ("xq", "q"):
        np.testing.assert_array_equal(req.matrix(L[k]).reshape(kept[L[k]].shape).view(np.int8), kept[L[k]].astype(np.int8))
    for k in ("ctx", "down"):
        np.testing.assert_array_equal(req.matrix(L[k]).reshape(kept[L[k]].shape).view(np.uint32), kept[L[k]].view(np.uint32))
    np.testing.assert_array_equal(y.view(np.uint32), want["out"].view(np.uint32))


def test_full_size_embedding_front_end_from_token_ids(orc, monkeypatch):
    """Benchmark configuration 5 from its token ids: ids uniform in [0, 30522) for 16 sequences of 384 tokens, word table
    [30522, 768] + position table + token-type row -> LayerNorm -> the first layer's quantized activations.  The lookup
    and the sums are bit-exact, the normalisation within its tolerance, the i8 levels behind it equal to the reference
    FakeQuantize of the device's own f32 values (one encoder layer: the other eleven repeat it and are covered by
    test_encoder_full_size_first_and_last_layer)"""
    from dldt_amd import builders
    monkeypatch.setenv("HIPIE_KEEP_F32", "1")
    B, S, H, V = 16, 384, 768, 30522
    g, meta = builders.bert_encoder(layers=1, hidden=H, heads=12, ffn=3072, batch=B, seq=S, seed=21, vocab=V)
    ids = np.random.default_rng(30522).integers(0, V, (B, S)).astype(np.int32)
    assert ids.max() > V - 50 and ids.min() < 50
    plan = g.compile()
    assert [s["type"] for s in plan.steps[:2]] == ["Gather", "MVN+FakeQuantize"]
    assert plan.inputs[0]["name"] == "input_ids" and plan.inputs[0]["shape"] == (B, S)
    req = plan.create_request()
    req.infer(ids)
    L = meta["layers"][0]
    device = {n: req.matrix(n) for n in meta["glue"] if n == meta["embedding_norm"]}
    _, kept = evaluate(orc, g.nodes, {"input_ids": ids}, keep=[meta["embeddings"], meta["embedding_norm"]],
                       targets=[meta["embedding_norm"]])
    emb = kept[meta["embeddings"]]
    np.testing.assert_array_equal(req.matrix(meta["embeddings"]).reshape(emb.shape).view(np.uint32), emb.view(np.uint32))
    w = kept[meta["embedding_norm"]]
    np.testing.assert_allclose(device[meta["embedding_norm"]].reshape(w.shape), w, rtol=1e-5, atol=4e-6)
    _, kept = evaluate(orc, g.nodes, {"input_ids": ids}, keep=[L["xq"]], override=device, targets=[L["xq"]])
    np.testing.assert_array_equal(req.matrix(L["xq"]).reshape(kept[L["xq"]].shape).view(np.int8), kept[L["xq"]].astype(np.int8))


def test_encoder_with_attention_mask(orc, monkeypatch):
    """additive mask [batch, 1, 1, seq] between the score Multiply and the Softmax: padded keys get no weight"""
    from dldt_amd import builders
    monkeypatch.setenv("HIPIE_KEEP_F32", "1")
    B, S, H = 2, 96, 128
    g, meta = builders.bert_encoder(layers=2, hidden=H, heads=2, ffn=256, batch=B, seq=S, seed=11, mask=True,
                                    ranges=dict(q=0.12, k=0.9, v=0.9, ctx=0.6))
    rng = np.random.default_rng(12)
    x = rng.normal(0, 1, (B, S, H)).astype(np.float32)
    mask = np.zeros((B, 1, 1, S), np.float32)
    mask[0, 0, 0, 70:] = -10000.0
    mask[1, 0, 0, 33:] = -10000.0
    plan = g.compile()
    assert [s["type"] for s in plan.steps].count("Attention") == 2 and len(plan.inputs) == 2
    req = plan.create_request()
    (y,) = req.infer(x, mask)
    device = {n: req.matrix(n) for n in meta["glue"]}
    keep = [n for L in meta["layers"] for n in L.values()]
    want, kept = evaluate(orc, g.nodes, {"hidden_states": x, "attention_mask": mask}, keep=keep, override=device)
    for li, L in enumerate(meta["layers"]):
        p = device[L["p"]].reshape(B, 2, S, S)
        assert p[0, :, :, 70:].max() == 0.0 and p[1, :, :, 33:].max() == 0.0
        w = kept[("oracle", L["p"])]
        np.testing.assert_allclose(p, w, rtol=3e-6, atol=1e-8, err_msg="layer %d" % li)
        for name in ("ctx", "attn", "down"):
            np.testing.assert_array_equal(req.matrix(L[name]).reshape(kept[L[name]].shape).view(np.uint32),
                                          kept[L[name]].view(np.uint32), err_msg="layer %d %s" % (li, name))
    np.testing.assert_array_equal(y.view(np.uint32), want["out"].view(np.uint32))


@pytest.mark.parametrize("seq,fuse", [(128, False), (448, True)])
def test_attention_mask_where_the_core_runs_as_separate_kernels(orc, monkeypatch, seq, fuse):
    """the same mask where the attention core is not one kernel (switched off, or a sequence longer than the fused
    kernel takes): MatMul -> Add(mask, numpy broadcasting over heads and queries) -> Softmax -> MatMul as steps of
    their own; the Add is one f32 addition and compared bit for bit, the rest as in the fused form"""
    from dldt_amd import builders
    monkeypatch.setenv("HIPIE_KEEP_F32", "1")
    monkeypatch.setenv("HIPIE_FUSE_ATTENTION", "1" if fuse else "0")
    B, S, H = 2, seq, 128
    g, meta = builders.bert_encoder(layers=1, hidden=H, heads=2, ffn=256, batch=B, seq=S, seed=13, mask=True,
                                    ranges=dict(q=0.12, k=0.9, v=0.9, ctx=0.6))
    rng = np.random.default_rng(14)
    x = rng.normal(0, 1, (B, S, H)).astype(np.float32)
    mask = np.zeros((B, 1, 1, S), np.float32)
    mask[0, 0, 0, S - 30:] = -10000.0
    mask[1, 0, 0, 33:] = -10000.0
    plan = g.compile()
    types = [s["type"] for s in plan.steps]
    assert types.count("Attention") == 0 and types.count("Add") == 1 and len(plan.inputs) == 2
    req = plan.create_request()
    (y,) = req.infer(x, mask)
    L = meta["layers"][0]
    masked = next(i for i, n in enumerate(g.nodes) if n["op"] == "Add" and meta_mask(g) in n["inputs"])
    device = {n: req.matrix(n) for n in meta["glue"]}
    want, kept = evaluate(orc, g.nodes, {"hidden_states": x, "attention_mask": mask}, keep=list(L.values()) + [masked], override=device)
    np.testing.assert_array_equal(req.matrix(masked).reshape(B, 2, S, S).view(np.uint32), kept[masked].view(np.uint32))
    p = device[L["p"]].reshape(B, 2, S, S)
    assert p[0, :, :, S - 30:].max() == 0.0 and p[1, :, :, 33:].max() == 0.0
    np.testing.assert_allclose(p, kept[("oracle", L["p"])], rtol=3e-6, atol=1e-8)
    for name in ("ctx", "attn", "down"):
        np.testing.assert_array_equal(req.matrix(L[name]).reshape(kept[L[name]].shape).view(np.uint32), kept[L[name]].view(np.uint32), err_msg=name)
    np.testing.assert_array_equal(y.view(np.uint32), want["out"].view(np.uint32))
    assert all(g.query())


def meta_mask(g):
    return next(i for i, n in enumerate(g.nodes) if n["op"] == "Parameter" and n["name"] == "attention_mask")


def test_encoder_full_size_first_and_last_layer(orc, monkeypatch):
    """Benchmark configuration 5 at its stated size (12 layers x 768, 12 heads, FFN 3072, sequence 384, batch 16):
    every integer segment of the first and the last layer (projections, attention, both FFN GEMMs with their
    dequantisation, residual and requantisation) equals the oracle's, which continues from the device's own value
    behind each tolerance-only op (Softmax, LayerNorm, Gelu) and, for the last layer, from the device's input of that
    layer; the glue ops of both layers are compared with what the oracle makes of the device's inputs to them."""
    from dldt_amd import builders
    monkeypatch.setenv("HIPIE_KEEP_F32", "1")
    B, S, H, NH, FF = 16, 384, 768, 12, 3072
    g, meta = builders.bert_encoder(layers=12, hidden=H, heads=NH, ffn=FF, batch=B, seq=S)
    x = np.random.default_rng(5).normal(0, 1, (B, S, H)).astype(np.float32)
    plan = g.compile()
    assert [s["type"] for s in plan.steps].count("Attention") == 12
    req = plan.create_request()
    (y,) = req.infer(x)
    assert np.isfinite(y).all()
    shape = dict(p=(B, NH, S, S), h1=(B, S, H), gelu=(B, S, FF), y=(B, S, H), scores=(B, NH, S, S), attn=(B, S, H),
                 up=(B, S, FF), down=(B, S, H))
    glue_input = dict(p="scores", h1="attn", gelu="up", y="down")
    for li in (0, 11):
        L = meta["layers"][li]
        mine = list(L.values())
        given = {L[n]: req.matrix(L[n]).reshape(shape[n]) for n in GLUE_TOL}
        if li > 0:
            prev = meta["layers"][li - 1]["y"]
            given[prev] = req.matrix(prev).reshape(B, S, H)
        _, kept = evaluate(orc, g.nodes, {"hidden_states": x}, keep=mine, override=given, targets=mine)
        for name in EXACT:
            if name == "pq":
                continue                                  # stays in registers inside the attention kernel
            w = kept[L[name]]
            have = req.matrix(L[name]).reshape(w.shape)
            if w.dtype == np.float32:
                np.testing.assert_array_equal(have.view(np.uint32), w.view(np.uint32), err_msg="layer %d %s" % (li, name))
            else:
                np.testing.assert_array_equal(have.view(np.int8), w.astype(np.int8), err_msg="layer %d %s" % (li, name))
        assert len(np.unique(kept[L["q"]])) > 60
        del kept
        for name, tol in GLUE_TOL.items():               # each glue op from the device's own input to it
            src = L[glue_input[name]]
            _, one = evaluate(orc, g.nodes, {"hidden_states": x}, keep=[L[name]],
                              override={src: req.matrix(src).reshape(shape[glue_input[name]])}, targets=[L[name]])
            w = one[L[name]]
            np.testing.assert_allclose(req.matrix(L[name]).reshape(w.shape), w, err_msg="layer %d %s" % (li, name), **tol)
    np.testing.assert_array_equal(y.reshape(-1, H).view(np.uint32),
                                  req.matrix(meta["layers"][11]["y"]).reshape(-1, H).view(np.uint32))


def test_weight_matmuls_with_activation_zero_points(orc):
    """u8 activations with zero points on the row-major path: the FakeQuantize behind a LayerNorm and the one in a
    GEMM's epilogue write u8 levels, and the Subtract that MatMulTransformation leaves behind each MatMul (zero
    point x column sums of the weights) starts the accumulators; everything behind the LayerNorm is bit-exact"""
    from dldt_amd import builders
    g, meta = builders.matmul_zero_point_net()
    assert all(z not in (0.0, 128.0) for z in meta["zero_points"])
    x = np.random.default_rng(8).normal(0, 1, (2, 48, 128)).astype(np.float32)
    plan = g.compile(config={"HIP_KEEP_F32": "YES"})
    types = [s["type"] for s in plan.steps]
    assert types.count("MatMul") == 2 and "MVN+FakeQuantize" in types
    req = plan.create_request()
    (y,) = req.infer(x)
    device = {meta["norm"]: req.matrix(meta["norm"])}
    want, kept = evaluate(orc, g.nodes, {"hidden_states": x}, keep=[meta["a0"], meta["a1"]], override=device)
    np.testing.assert_allclose(device[meta["norm"]].reshape(kept[("oracle", meta["norm"])].shape), kept[("oracle", meta["norm"])],
                               rtol=1e-5, atol=4e-6)
    for name in ("a0", "a1"):
        w = kept[meta[name]]
        assert w.dtype == np.uint8 and w.min() == 0 and w.max() == 255
        have = req.matrix(meta[name]).reshape(w.shape)          # stored as level - 128, read back as levels
        assert have.dtype == np.uint8
        np.testing.assert_array_equal(have, w, err_msg=name)
    np.testing.assert_array_equal(y.view(np.uint32), want["out"].view(np.uint32))
    # without the kept f32 values: the same bits
    (y2,) = g.compile().create_request().infer(x)
    np.testing.assert_array_equal(y2.view(np.uint32), y.view(np.uint32))
