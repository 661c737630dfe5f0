"""One BERT-base style encoder layer in its post-LPT form (benchmark configuration 5), composed on the host
from the operator-level C ABI: per-tensor symmetric i8 activations, per-channel i8 weights, int8 MFMA
GEMMs with fused dequantisation, fp32 softmax / LayerNorm / GELU.

Graph of one layer (what LowPrecision leaves for MatMulTransformation, mat_mul.cpp:81-171, with the
bias moved in front of the dequantisation Multiply by AddTransformation, add.cpp:125-153):

    xq   = FQ_i8(x)                                   per tensor, scale sx
    qkv  = FQ_i8((xq . Wqkv' + b') * (sx * sw[c]))    one GEMM, requantised per Q/K/V segment
    s    = (q . k^T) * (sq * sk)                      per (batch, head); 1/sqrt(d) is folded into Wq
    p    = Softmax(s);  pq = FQ_i8(p)
    ctx  = (pq . v) * (sp * sv)                       v transposed to [d, S] (Transpose node)
    a    = ((FQ_i8(ctx) . Wo' + b') * scale) + x;     h1 = LayerNorm(a)
    f    = GELU((FQ_i8(h1) . W1' + b') * scale)
    o    = ((FQ_i8(f) . W2' + b') * scale) + h1;      y = LayerNorm(o)

Every tensor a test may want is kept in ``EncoderLayer.t`` after ``run``.
"""
import numpy as np

from .ops import (BatchedMatMul, Convolution, FakeQuantize, gelu, make_epilogue, matmul_strided, mvn, softmax,
                  transpose_bytes)
from .tensor import DeviceTensor

F32, I8 = 10, 50


def sym_i8_range(absmax):
    """(in_low, in_high, scale) of a symmetric signed FakeQuantize with 256 levels whose dequantisation
    scale is absmax / 127 (levels -128 .. 127)."""
    s = np.float32(absmax) / np.float32(127)
    return np.float32(-128) * s, np.float32(127) * s, s


def quantize_weights(w):
    """Per-output-channel symmetric i8 (255 levels, -127 .. 127): the constant-folded weight
    FakeQuantize of weightable_layer_transformation.cpp:285-321."""
    m = np.abs(w).max(axis=1).astype(np.float32)
    sw = m / np.float32(127)
    q = np.clip(np.rint(w / sw[:, None]), -127, 127).astype(np.int8)
    return q, sw.astype(np.float32)


class EncoderLayer:
    def __init__(self, hidden=768, heads=12, ffn=3072, batch=16, seq=384, seed=20211, ranges=None):
        assert hidden % heads == 0 and hidden // heads == 64, "head dimension 64 (one MFMA K step)"
        assert seq % 64 == 0, "the context MatMul reduces over the sequence: multiple of 64"
        self.H, self.NH, self.FF, self.B, self.S = hidden, heads, ffn, batch, seq
        self.T = batch * seq
        rng = np.random.default_rng(seed)
        n = lambda *shape: rng.normal(0, 0.02, shape).astype(np.float32)
        H, FF = hidden, ffn
        self.w = {"qkv": n(3 * H, H), "o": n(H, H), "up": n(FF, H), "down": n(H, FF)}
        self.w["qkv"][:H] *= np.float32(0.125)            # 1/sqrt(64) folded into the query projection
        self.b = {"qkv": n(3 * H), "o": n(H), "up": n(FF), "down": n(H)}
        self.ln = [(1 + n(H), n(H)), (1 + n(H), n(H))]
        # activation ranges (absmax per quantized tensor); a caller may pass calibrated ones
        self.r = dict(x=4.0, q=1.2, k=3.0, v=3.0, p=1.0, ctx=1.0, h1=4.0, g=3.0)
        if ranges:
            self.r.update(ranges)
        self.wq, self.sw = {}, {}
        for k, w in self.w.items():
            self.wq[k], self.sw[k] = quantize_weights(w)
        self._build()

    # ------------------------------------------------------------------------------------------
    def _fq(self, key):
        il, ih, s = sym_i8_range(self.r[key])
        return FakeQuantize(1, 256, il, ih, -128.0, 127.0), s

    def _linear(self, name, x_scale, in_dt, epi_extra):
        """1x1 convolution over [T, K]: (acc + b / (sx * sw)) * (sx * sw) [...]"""
        scale = (np.float32(x_scale) * self.sw[name]).astype(np.float32)
        bias = (self.b[name] / scale).astype(np.float32)          # swapMultiplyAndAdd: b / a in f32
        self.c[name] = dict(scale=scale, bias=bias)
        epi = make_epilogue(bias=bias, scale=scale, **epi_extra)
        w = self.wq[name]
        return Convolution(w.reshape(w.shape[0], w.shape[1], 1, 1), in_dt, epilogue=epi)

    def _build(self):
        import torch
        T, H, FF, B, S, NH = self.T, self.H, self.FF, self.B, self.S, self.NH
        self.c = {}
        self.fq, self.s = {}, {}
        for k in ("x", "p", "ctx", "h1", "g"):
            self.fq[k], self.s[k] = self._fq(k)
        for k in ("q", "k", "v"):
            _, _, self.s[k] = sym_i8_range(self.r[k])
        dt = lambda c, dtype: DeviceTensor(1, 1, T, c, dtype)
        self.d = dict(xq=dt(H, I8), qkv=dt(3 * H, I8), ctxq=dt(H, I8), x=dt(H, F32), attn=dt(H, F32), h1=dt(H, F32),
                      h1q=dt(H, I8), f=dt(FF, F32), gq=dt(FF, I8), o=dt(H, F32))
        # QKV: one GEMM, requantised per segment
        il = np.concatenate([np.full(H, sym_i8_range(self.r[k])[0], np.float32) for k in ("q", "k", "v")])
        ih = np.concatenate([np.full(H, sym_i8_range(self.r[k])[1], np.float32) for k in ("q", "k", "v")])
        self.c["qkv_fq"] = (il, ih)
        self.lin = {
            "qkv": self._linear("qkv", self.s["x"], self.d["xq"], dict(out_dtype=I8, fq=(256, il, ih, -128.0, 127.0))),
            "o": self._linear("o", self.s["ctx"], self.d["ctxq"], dict(residual_dtype=F32, out_dtype=F32)),
            "up": self._linear("up", self.s["h1"], self.d["h1q"], dict(out_dtype=F32)),
            "down": self._linear("down", self.s["g"], self.d["gq"], dict(residual_dtype=F32, out_dtype=F32)),
        }
        self.c["scores_scale"] = np.float32(self.s["q"]) * np.float32(self.s["k"])
        self.c["ctx_scale"] = np.float32(self.s["p"]) * np.float32(self.s["v"])
        self.mm_scores = BatchedMatMul(64, S, make_epilogue(scale=[self.c["scores_scale"]], out_dtype=F32))
        self.mm_ctx = BatchedMatMul(S, 64, make_epilogue(scale=[self.c["ctx_scale"]], out_dtype=F32))
        dev = "cuda"
        self.scores = torch.empty((B, NH, S, S), dtype=torch.float32, device=dev)
        self.pq = torch.empty((B, NH, S, S), dtype=torch.int8, device=dev)
        self.vt = torch.empty((B, NH, 64, S), dtype=torch.int8, device=dev)
        self.ctx = torch.empty((T, H), dtype=torch.float32, device=dev)
        self.g = [(torch.from_numpy(g).to(dev), torch.from_numpy(b).to(dev)) for g, b in self.ln]

    @staticmethod
    def _flat(d):
        """[T, C] torch view of a channel-dense DeviceTensor."""
        assert d.cs == d.c and d.halo == 0
        return d.interior().view(d.w, d.c)

    def run(self, x):
        """x: torch f32 [B, S, H] on the device.  Returns y f32 [B, S, H]; intermediates in self.t."""
        B, S, H, NH, T = self.B, self.S, self.H, self.NH, self.T
        d, flat = self.d, self._flat
        flat(d["x"]).copy_(x.reshape(T, H))
        q4 = lambda t, c: t.view(1, 1, T, c)
        self.fq["x"].run_q8(q4(flat(d["x"]), H), "i8", "nchw", out=q4(flat(d["xq"]), H))
        self.lin["qkv"].run(d["xq"], d["qkv"])
        qkv = flat(d["qkv"])
        base = qkv.data_ptr()
        # (sequence, head) is a two-level batch inside [T, 3H]: heads 64 columns apart, sequences S rows apart
        matmul_strided(self.mm_scores, base, 3 * H, 64, base + H, 3 * H, 64, self.scores.data_ptr(), S, S * S, S, NH,
                       batch_outer=B, outer_a=S * 3 * H, outer_b=S * 3 * H, outer_o=NH * S * S)
        transpose_bytes(base + 2 * H, 3 * H, 64, self.vt.data_ptr(), S, 64 * S, S, 64, NH,
                        batch_outer=B, outer_src=S * 3 * H, outer_dst=NH * 64 * S)
        p = softmax(self.scores.view(B * NH * S, S))
        self.fq["p"].run_q8(p.view(1, 1, B * NH * S, S), "i8", "nchw", out=self.pq.view(1, 1, B * NH * S, S))
        # context written straight into [T, H] at its head's columns
        matmul_strided(self.mm_ctx, self.pq.data_ptr(), S, S * S, self.vt.data_ptr(), S, 64 * S, self.ctx.data_ptr(), H, 64,
                       S, NH, batch_outer=B, outer_a=NH * S * S, outer_b=NH * 64 * S, outer_o=S * H)
        self.fq["ctx"].run_q8(q4(self.ctx, H), "i8", "nchw", out=q4(flat(d["ctxq"]), H))
        self.lin["o"].run(d["ctxq"], d["attn"], d["x"])
        h1 = mvn(flat(d["attn"]), gamma=self.g[0][0], beta=self.g[0][1])
        flat(d["h1"]).copy_(h1)
        self.fq["h1"].run_q8(q4(h1, H), "i8", "nchw", out=q4(flat(d["h1q"]), H))
        self.lin["up"].run(d["h1q"], d["f"])
        gl = gelu(flat(d["f"]))
        self.fq["g"].run_q8(q4(gl, self.FF), "i8", "nchw", out=q4(flat(d["gq"]), self.FF))
        self.lin["down"].run(d["gq"], d["o"], d["h1"])
        y = mvn(flat(d["o"]), gamma=self.g[1][0], beta=self.g[1][1])
        self.t = dict(xq=flat(d["xq"]), qkv=qkv, scores=self.scores, p=p, pq=self.pq, vt=self.vt, ctx=self.ctx,
                      ctxq=flat(d["ctxq"]), attn=flat(d["attn"]), h1=h1, h1q=flat(d["h1q"]), f=flat(d["f"]), gelu=gl,
                      gq=flat(d["gq"]), o=flat(d["o"]), y=y)
        return y.view(B, S, H)

    def macs(self):
        T, H, FF = self.T, self.H, self.FF
        return T * (4 * H * H + 2 * H * FF) + 2 * self.B * self.NH * self.S * self.S * 64
