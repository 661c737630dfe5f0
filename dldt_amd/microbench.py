#!/usr/bin/env python3
"""Kernel timings at the shapes of the five benchmark configurations, against each kernel's roofline.

    python -m dldt_amd.microbench            # all rows, markdown table on stdout
    python -m dldt_amd.microbench encoder    # only the 12-layer encoder graph of config 5

Rows: config 1 (one quantized 3x3 convolution block, batch 1), config 2 (per-channel FakeQuantize of
[32,256,56,56]), config 3 (ResNet-50 v1.5 INT8, batch 1 and 64), config 4 (MobileNetV2 INT8, batch 64:
whole graph, its depthwise and pointwise kernels), config 5 (one BERT-base encoder layer at batch 16,
sequence 384: the int8 GEMMs and the fp32 softmax / LayerNorm / GELU kernels, each on its own; then the
12-layer encoder as one graph through the planner).
Inputs are resident in HBM, times are HIP-event averages over back-to-back launches.
"""
import sys

import numpy as np

INT8_PEAK_TOPS = 5000.0
HBM_PEAK_GBS = 8000.0
F32, U8, I8, I32, U8B = 10, 40, 50, 70, 41


def _time(fn, reps=30, warm=5):
    import torch
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(reps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / reps * 1e3   # us


def _launches(plan):
    """kernels one inference of the plan enqueues (a step may run two)"""
    return sum(int(plan.step_rt_info(i, "kernels")) for i in range(len(plan.steps)))


def _graph_time(g, reps=20, warm=5):
    """(us per inference, plan) of a compiled graph, kernels only, on the request's stream."""
    import torch
    plan = g.compile(0)
    req = plan.create_request()
    ins, outs = req.device_buffers()
    for t in ins:
        t.copy_(torch.rand(t.shape, device="cuda"))
    stream = torch.cuda.ExternalStream(req.stream)
    torch.cuda.synchronize()
    for _ in range(warm):
        req.enqueue(ins, outs)
    stream.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record(stream)
    for _ in range(reps):
        req.enqueue(ins, outs)
    b.record(stream)
    stream.synchronize()
    return a.elapsed_time(b) / reps * 1e3, plan


def _throughput_time(plan, nreq=3, reps=60, warm=9):
    """us per inference with nreq requests of one plan kept in flight on their own streams."""
    import time
    import torch
    reqs = [plan.create_request() for _ in range(nreq)]
    bufs = [r.device_buffers() for r in reqs]
    for ins, _ in bufs:
        for t in ins:
            t.copy_(torch.rand(t.shape, device="cuda"))
    streams = [torch.cuda.ExternalStream(r.stream) for r in reqs]
    torch.cuda.synchronize()
    for i in range(warm):
        reqs[i % nreq].enqueue(*bufs[i % nreq])
    for st in streams:
        st.synchronize()
    t0 = time.perf_counter()
    for i in range(reps):
        reqs[i % nreq].enqueue(*bufs[i % nreq])
    for st in streams:
        st.synchronize()
    return (time.perf_counter() - t0) / reps * 1e6


def _best_variant(conv, run, tiles=(0, 1, 4, 5, 10, 11, 12, 18, 19, 20, 21, 22)):
    """(us, variant): the fastest of the kernel variants that take the layer, as the load-time tuner would choose"""
    from . import HipieError
    best = None
    for tile in tiles:
        try:
            conv.set_tile(tile)
        except HipieError:
            continue
        if conv.get_tile() != tile:
            continue
        us = _time(run)
        if best is None or us < best[0]:
            best = (us, tile)
    conv.set_tile(best[1])
    return best


def _row(name, us, macs=0, bytes_=0, bound=None):
    tops = 2.0 * macs / us / 1e6 if macs else 0.0
    gbs = bytes_ / us / 1e3 if bytes_ else 0.0
    if bound is None:
        bound = "mfma" if macs and (tops / INT8_PEAK_TOPS >= gbs / HBM_PEAK_GBS) else "hbm"
    frac = tops / INT8_PEAK_TOPS if bound == "mfma" else gbs / HBM_PEAK_GBS
    return {"row": name, "us": us, "TOP/s": tops, "GB/s": gbs, "bound": bound, "frac": frac}


def config1():
    from . import builders
    g, _, _ = builders.conv_block()
    us, plan = _graph_time(g)
    macs = sum(s["macs"] for s in plan.steps)
    return [_row("cfg1 FQ + 3x3 conv 64->64 @56x56 + bias + ReLU, batch 1 (3 launches)", us, macs=macs,
                 bytes_=200704 * 4 + 200704 + 36864 + 802816)]


def config2():
    import torch
    from . import FakeQuantize
    n, c, h, w = 32, 256, 56, 56
    rng = np.random.default_rng(2)
    mu = rng.uniform(-0.5, 0.5, c).astype(np.float32)
    x = torch.randn((n, c, h, w), device="cuda") + torch.from_numpy(mu).cuda().view(1, c, 1, 1)
    fq = FakeQuantize(c, 256, mu - 3, mu + 3, 0.0, 255.0)
    y8 = torch.empty(x.shape, dtype=torch.uint8, device="cuda")
    yf = torch.empty_like(x)
    yn = torch.empty((n, h, w, c), dtype=torch.int8, device="cuda")
    e = x.numel()
    return [
        _row("cfg2 FakeQuantize [32,256,56,56] per-channel, f32 -> u8 levels (NCHW)",
             _time(lambda: fq.run_q8(x, "u8", "nchw", out=y8)), bytes_=5 * e),
        _row("cfg2 same, f32 -> u8 levels NHWC (graph entry form)",
             _time(lambda: fq.run_q8(x, "u8b", "nhwc", c, out=yn)), bytes_=5 * e),
        _row("cfg2 same, f32 -> f32 (the operator as specified)", _time(lambda: fq.run_f32(x, out=yf)), bytes_=8 * e),
    ]


def config3():
    from . import builders
    rows = []
    for batch in (1, 64):
        g, meta = builders.resnet50(batch=batch, res=224)
        us, plan = _graph_time(g)
        r = _row("cfg3 ResNet-50 v1.5 INT8 batch %d, whole graph (%d launches)" % (batch, _launches(plan)), us,
                 macs=meta["macs_per_image"] * batch, bytes_=sum(s["bytes"] for s in plan.steps), bound="mfma")
        r["images/s"] = batch / us * 1e6
        rows.append(r)
        if batch > 1:
            us3 = _throughput_time(plan)
            r = _row("cfg3 ResNet-50 v1.5 INT8 batch %d, three requests in flight" % batch, us3,
                     macs=meta["macs_per_image"] * batch, bytes_=sum(s["bytes"] for s in plan.steps), bound="mfma")
            r["images/s"] = batch / us3 * 1e6
            rows.append(r)
    return rows


def config4():
    import torch
    from . import builders, Convolution, DeviceTensor, make_epilogue
    g, meta = builders.mobilenet_v2(batch=64, res=224)
    us, plan = _graph_time(g)
    r = _row("cfg4 MobileNetV2-1.0 INT8 batch 64, whole graph (%d launches)" % _launches(plan), us,
             macs=meta["macs_per_image"] * 64, bytes_=sum(s["bytes"] for s in plan.steps))
    r["images/s"] = 64 / us * 1e6
    rows = [r]
    us3 = _throughput_time(plan)
    r = _row("cfg4 MobileNetV2-1.0 INT8 batch 64, three requests in flight", us3, macs=meta["macs_per_image"] * 64,
             bytes_=sum(s["bytes"] for s in plan.steps))
    r["images/s"] = 64 / us3 * 1e6
    rows.append(r)
    rng = np.random.default_rng(4)
    # every distinct depthwise layer of MobileNetV2 with its own tail (bias, scale, ReLU6, FakeQuantize(0, 6)),
    # both kernel variants: 0 = from registers, 1 = through an LDS patch with the window sliding in registers
    for c, hw, stride in ((32, 112, 1), (96, 112, 2), (144, 56, 1), (144, 56, 2), (192, 28, 1), (192, 28, 2), (384, 14, 1),
                          (576, 14, 1), (576, 14, 2), (960, 7, 1)):
        cs = -(-c // 16) * 16
        xin = DeviceTensor(64, hw, hw, c, U8B, halo=1)
        xin.interior().copy_(torch.randint(-128, 127, xin.interior().shape, dtype=torch.int8, device="cuda"))
        w = rng.integers(-127, 128, (c, 1, 1, 3, 3)).astype(np.int8)
        fq = (256, 0.0, np.float32(6.0), 0.0, 255.0)
        conv = Convolution(w, xin, (stride, stride), (1, 1), (1, 1), (1, 1),
                           make_epilogue(bias=np.zeros(c, np.float32), scale=np.full(c, 2e-4, np.float32), activation="clamp",
                                         clamp=(0.0, 6.0), out_dtype=U8B, fq=fq))
        oh = (hw + 2 - 3) // stride + 1
        out = DeviceTensor(64, oh, oh, c, U8B)
        for variant in (0, 1, 2):
            conv.set_tile(variant)
            rows.append(_row("cfg4 depthwise 3x3 s%d C=%d @%dx%d batch 64, variant %d" % (stride, c, hw, hw, variant),
                             _time(lambda: conv.run(xin, out)), macs=64 * oh * oh * c * 9,
                             bytes_=64 * (hw * hw + oh * oh) * cs + 9 * c, bound="hbm"))
    return rows


def config5():
    import torch
    from . import BatchedMatMul, Convolution, DeviceTensor, make_epilogue, softmax, mvn, gelu
    B, S, H, NH, FF = 16, 384, 768, 12, 3072
    T = B * S
    rng = np.random.default_rng(5)
    rows = []
    layer_us = 0.0

    def linear(name, k, n, out_dtype, count=1):
        nonlocal layer_us
        xin = DeviceTensor(1, 1, T, k, I8)
        xin.interior().copy_(torch.randint(-128, 127, xin.interior().shape, dtype=torch.int8, device="cuda"))
        w = rng.integers(-127, 128, (n, k, 1, 1)).astype(np.int8)
        if out_dtype == F32:
            ep = make_epilogue(bias=np.zeros(n, np.float32), scale=np.full(n, 1e-4, np.float32), out_dtype=F32)
        else:
            ep = make_epilogue(bias=np.zeros(n, np.float32), out_dtype=I8,
                               fq=(256, np.full(n, -128e3, np.float32), np.full(n, 127e3, np.float32), -128.0, 127.0))
        conv = Convolution(w, xin, epilogue=ep)
        out = DeviceTensor(1, 1, T, n, out_dtype)
        us, variant = _best_variant(conv, lambda: conv.run(xin, out))
        layer_us += us * count
        rows.append(_row("cfg5 %s [%d,%d]x[%d,%d] -> %s (variant %d)" % (name, T, k, k, n, "f32" if out_dtype == F32 else "i8", variant), us,
                         macs=T * k * n, bytes_=T * k + k * n + T * n * (4 if out_dtype == F32 else 1), bound="mfma"))

    linear("QKV projection", H, 3 * H, I8)
    linear("attention output projection", H, H, F32)
    linear("FFN up", H, FF, F32)
    linear("FFN down", FF, H, F32)

    def attention(name, m, k, n):
        nonlocal layer_us
        a = torch.randint(-128, 127, (B * NH, m, k), dtype=torch.int8, device="cuda")
        bt = torch.randint(-128, 127, (B * NH, n, k), dtype=torch.int8, device="cuda")
        mm = BatchedMatMul(k, n, make_epilogue(scale=[1e-3], out_dtype=F32))
        out = torch.empty((B * NH, m, n), dtype=torch.float32, device="cuda")
        us = _time(lambda: mm.run(a, bt, out), reps=10, warm=3)
        layer_us += us
        rows.append(_row("cfg5 %s %dx[%d,%d]x[%d,%d] -> f32" % (name, B * NH, m, k, k, n), us,
                         macs=B * NH * m * k * n, bytes_=B * NH * (m * k + n * k + 4 * m * n)))

    attention("attention scores", S, 64, S)
    attention("attention context", S, S, 64)

    def glue(name, fn, x, passes):
        nonlocal layer_us
        us = _time(lambda: fn(x), reps=10, warm=3)
        layer_us += us * (2 if name.startswith("LayerNorm") else 1)
        rows.append(_row("cfg5 %s %s f32" % (name, list(x.shape)), us, bytes_=passes * 4 * x.numel(), bound="hbm"))

    glue("softmax", softmax, torch.randn((B * NH * S, S), device="cuda"), 2)
    gamma, beta = torch.ones(H, device="cuda"), torch.zeros(H, device="cuda")
    glue("LayerNorm (MVN, gamma, beta)", lambda t: mvn(t, gamma=gamma, beta=beta), torch.randn((T, H), device="cuda"), 2)
    glue("GELU (erf)", gelu, torch.randn((T, FF), device="cuda"), 2)
    # the attention core in one kernel: scores, softmax, requantisation, context (heads sliced out of [T, 3H])
    from .ops import Attention
    qkv = torch.randint(-128, 128, (B, S, 3, NH, 64), dtype=torch.int8, device="cuda")
    q, k, v = (qkv[:, :, i].permute(0, 2, 1, 3) for i in range(3))
    att = Attention(S, 64, 0.0007, 0.02 / 127, (-128.0 / 127, 1.0, -128, 256), out_fq=(-0.5, 0.5 * 127 / 128, -128, 256))
    ctx = torch.empty((B, NH, S, 64), dtype=torch.int8, device="cuda")
    us = _time(lambda: att.run(q, k, v, out=ctx), reps=10, warm=3)
    rows.append(_row("cfg5 fused attention %dx[%d,64]: scores, softmax, FakeQuantize, context -> i8" % (B * NH, S), us,
                     macs=2 * B * NH * S * S * 64, bytes_=4 * B * NH * S * 64))
    r = _row("cfg5 one encoder layer, sum of the separate kernels above (LayerNorm twice)", layer_us,
             macs=T * (4 * H * H + 2 * H * FF) + 2 * B * NH * S * S * 64, bound="mfma")
    r["sequences/s (12 layers, these kernels only)"] = B / (12 * layer_us) * 1e6
    rows.append(r)
    return rows + config5_graph()


def config5_graph():
    """the 12-layer encoder as a post-LPT graph through the planner (graph-level C ABI)"""
    from . import builders
    B, S, H, NH, FF = 16, 384, 768, 12, 3072
    rows = []
    g, meta = builders.bert_encoder(layers=12, hidden=H, heads=NH, ffn=FF, batch=B, seq=S)
    us, plan = _graph_time(g, reps=5, warm=2)
    r = _row("cfg5 BERT-base encoder, 12 layers, batch %d x %d tokens, one request (%d launches)" % (B, S, _launches(plan)),
             us, macs=meta["macs"], bytes_=sum(s["bytes"] for s in plan.steps), bound="mfma")
    r["sequences/s"] = B / us * 1e6
    rows.append(r)
    us3 = _throughput_time(plan, reps=12, warm=3)
    r = _row("cfg5 BERT-base encoder, 12 layers, three requests in flight", us3, macs=meta["macs"],
             bytes_=sum(s["bytes"] for s in plan.steps), bound="mfma")
    r["sequences/s"] = B / us3 * 1e6
    rows.append(r)
    return rows


def vendor_gemm():
    """The int8 GEMM of the vendor library (hipBLASLt behind torch._int_mm: plain [M, K] x [K, N] -> i32, no
    epilogue, no convolution addressing) on the GEMM shapes of ResNet-50 batch-64 layers and of the encoder's FFN,
    beside this library's convolution / MatMul kernels on the same layers with raw i32 output (the best of the kernel
    variants that take the layer, as the load-time tuner would choose)."""
    import numpy as np
    import torch
    from . import Convolution, DeviceTensor
    from .tensor import I32, U8B
    layers = [("ResNet stage-1 1x1 64->256 @56x56", 64, 64, 56, 256, 1),
              ("ResNet stage-2 3x3 128->128 @28x28", 64, 128, 28, 128, 3),
              ("ResNet stage-3 3x3 256->256 @14x14", 64, 256, 14, 256, 3),
              ("ResNet stage-3 1x1 1024->256 @14x14", 64, 1024, 14, 256, 1),
              ("ResNet stage-3 1x1 256->1024 @14x14", 64, 256, 14, 1024, 1),
              ("ResNet stage-4 3x3 512->512 @7x7", 64, 512, 7, 512, 3),
              ("encoder FFN up 768->3072, 6144 rows", 1, 768, 0, 3072, 1),
              ("encoder FFN down 3072->768, 6144 rows", 1, 3072, 0, 768, 1)]
    rows = []
    rng = np.random.default_rng(1)
    for name, n, c, hw, oc, k in layers:
        h, w_ = (hw, hw) if hw else (1, 6144)
        M, K = n * h * w_, c * k * k
        a = torch.randint(-128, 127, (M, K), dtype=torch.int8, device="cuda")
        b = torch.randint(-128, 127, (K, oc), dtype=torch.int8, device="cuda")
        us_vendor = _time(lambda: torch._int_mm(a, b))
        del a, b
        x = DeviceTensor(n, h, w_, c, U8B, halo=k // 2)
        wts = rng.integers(-127, 128, (oc, c, k, k)).astype(np.int8)
        conv = Convolution(wts, x, (1, 1), (1, 1), (k // 2, k // 2), (k // 2, k // 2))
        out = DeviceTensor(n, h, w_, oc, I32)
        best = _best_variant(conv, lambda: conv.run(x, out))
        rows.append(_row("%s: vendor GEMM [%d, %d] x [%d, %d] -> i32" % (name, M, K, K, oc), us_vendor, macs=M * K * oc, bound="mfma"))
        rows.append(_row("%s: this library, i32 output (variant %d)" % (name, best[1]), best[0], macs=M * K * oc, bound="mfma"))
    M = 8192
    a = torch.randint(-128, 127, (M, M), dtype=torch.int8, device="cuda")
    b = torch.randint(-128, 127, (M, M), dtype=torch.int8, device="cuda")
    rows.append(_row("vendor GEMM [8192, 8192] x [8192, 8192] -> i32 (what a large square problem reaches)",
                     _time(lambda: torch._int_mm(a, b), reps=10, warm=2), macs=M * M * M, bound="mfma"))
    del a, b
    x = DeviceTensor(1, 1, M, M, U8B)
    conv = Convolution(rng.integers(-127, 128, (M, M, 1, 1)).astype(np.int8), x)
    out = DeviceTensor(1, 1, M, M, I32)
    us, tile = _best_variant(conv, lambda: conv.run(x, out), tiles=(0, 4, 5, 10, 18, 19, 20, 21, 22))
    rows.append(_row("this library on the same problem (1 x 1 convolution, 8192 channels, 8192 pixels, variant %d)" % tile, us,
                     macs=M * M * M, bound="mfma"))
    return rows


def lds_rate():
    """LDS reads alone and mixed one to one with matrix instructions, 1 to 4 waves per SIMD (the GB/s column is the whole
    device by HIP events; bytes per clock and compute unit divide it by the core clock a wave measured meanwhile)"""
    import ctypes
    from ._lib import check, lib
    rows = []
    for with_mfma in (0, 1):
        for waves in (1, 2, 4):
            bpc, gbs = ctypes.c_double(), ctypes.c_double()
            check(lib().hipie_probe_lds_rate(0, 20000, waves, with_mfma, ctypes.byref(bpc), ctypes.byref(gbs)))
            what = "ds_read_b128 + one matrix instruction per read" if with_mfma else "ds_read_b128 alone"
            rows.append({"row": "%s, %d wave(s) per SIMD: %.1f B/clk per compute unit" % (what, waves, bpc.value),
                         "us": 0.0, "TOP/s": gbs.value * 64e-6 * 1e3 if with_mfma else 0.0, "GB/s": gbs.value, "bound": "lds",
                         "frac": bpc.value / 128.0})
    return rows


def mfma_rate():
    """the matrix pipe alone: every SIMD issuing int8 matrix instructions from registers, 1 to 4 waves per SIMD"""
    import ctypes
    from ._lib import check, lib
    rows = []
    for waves in (1, 2, 4):
        for iters in (20000, 200000):
            tops, ms = ctypes.c_double(), ctypes.c_double()
            check(lib().hipie_probe_mfma_rate(0, iters, waves, ctypes.byref(tops), ctypes.byref(ms)))
            r = {"row": "int8 matrix instructions from registers, %d wave(s) per SIMD, %.1f ms" % (waves, ms.value),
                 "us": ms.value * 1e3, "TOP/s": tops.value, "GB/s": 0.0, "bound": "mfma", "frac": tops.value / INT8_PEAK_TOPS}
            rows.append(r)
    return rows


def main():
    import torch
    assert torch.cuda.is_available(), "microbench needs a GPU"
    which = sys.argv[1:] or ["1", "2", "3", "4", "5"]
    table = {"1": config1, "2": config2, "3": config3, "4": config4, "5": config5, "encoder": config5_graph, "vendor": vendor_gemm, "mfma": mfma_rate, "lds": lds_rate}
    print("| kernel / graph | us | TOP/s | GB/s | bound | fraction of peak | notes |")
    print("|---|---|---|---|---|---|---|")
    for k in which:
        for r in table[k]():
            extra = ", ".join("%s %.0f" % (n, v) for n, v in r.items()
                              if n not in ("row", "us", "TOP/s", "GB/s", "bound", "frac"))
            print("| %s | %.1f | %.1f | %.0f | %s | %.3f | %s |" % (r["row"], r["us"], r["TOP/s"], r["GB/s"], r["bound"],
                                                                  r["frac"], extra))
            sys.stdout.flush()


if __name__ == "__main__":
    main()
