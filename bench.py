#!/usr/bin/env python3
"""ResNet-50 v1.5 INT8 inference throughput on one MI355X (the headline benchmark).

One step = one batch-64 inference of the post-LPT graph (entry FakeQuantize, 53 fused int8 MFMA
convolutions + FC, pools, exit), kernels only, inputs resident in HBM.  Like the reference's
benchmark_app in throughput mode (samples/benchmark_app/main.cpp: nireq asynchronous requests kept in
flight), the timed steps are issued round-robin over --requests infer requests, each with its own
stream and activation arena; --requests 1 is the latency mode, also measured and reported.
Prints one JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

INT8_PEAK_TOPS = 5000.0   # MI355X dense int8 MFMA, TOP/s
HBM_PEAK_GBS = 8000.0
# HBM bytes per convolution/FC launch at batch 64, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of
# this script (profiles/conv_kernels_resnet50_b64.md: 2.0 x FETCH_SIZE + 1.0 x WRITE_SIZE, factors
# calibrated on copies of known size in the same runs)
MEASURED_TRAFFIC_BYTES_PER_LAUNCH_B64 = 34.8e6


def cpu_baseline(batch_images, budget_s=20.0):
    """The oracle (C restatement of the reference kernels, OpenMP over host cores) evaluating the
    same post-LPT ResNet-50 graph on a bounded sample of images."""
    import numpy as np
    import oracle
    from interp import evaluate
    from dldt_amd import builders
    orc = oracle.require_ops()
    cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    g, _ = builders.resnet50(batch=1, res=224)
    x = np.random.default_rng(5).uniform(0, 1, (1, 3, 224, 224)).astype(np.float32)
    t0 = time.perf_counter()
    first, _ = evaluate(orc, g.nodes, {"data": x}, keep=[])
    one = time.perf_counter() - t0
    n = 1
    total = one
    while total + one < budget_s and n < batch_images:
        t0 = time.perf_counter()
        evaluate(orc, g.nodes, {"data": x}, keep=[])
        total += time.perf_counter() - t0
        n += 1
    return {"value": n / total, "unit": "images/sec", "cores": cores, "kind": "port",
            "sample": "%d image(s) of ResNet-50 v1.5 INT8 224x224 through oracle/ngraph_ops.c "
                      "(scalar int32 reference loops, OpenMP over batch x output channels), %.1f s" % (n, total)}, \
        x, first["logits"]


def parity_check(plan, batch, x, want):
    """The oracle's image as image 0 of one inference of the benchmarked plan (the other images random):
    its dequantised f32 logits against the oracle's, as the deviation relative to the output range and
    as top-1 agreement.  Integer-exact kernels and the same f32 epilogue make them equal bit for bit."""
    import numpy as np
    xb = np.random.default_rng(11).uniform(0, 1, (batch,) + x.shape[1:]).astype(np.float32)
    xb[0] = x[0]
    (y,) = plan.create_request().infer(xb)
    got, ref = y[0].astype(np.float64), want[0].astype(np.float64)
    rng_out = float(ref.max() - ref.min()) or 1.0
    return {"against": "oracle (reference ops on the post-LPT graph), image 0 of a batch-%d inference" % batch,
            "bit_exact": bool(np.array_equal(y[0].view(np.uint32), want[0].view(np.uint32))),
            "max_abs_over_output_range": float(np.abs(got - ref).max() / rng_out),
            "top1_agreement": float(int(np.argmax(got)) == int(np.argmax(ref))), "images": 1}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=240)
    ap.add_argument("--warmup", type=int, default=24)
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--requests", type=int, default=3,
                    help="infer requests in flight, one stream each (HIP gives a process 4 hardware queues here and the "
                         "default stream holds one: 3 ran 15 % faster than 4)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU (infer requests are independent, so more GPUs would each "
                 "run their own plan and requests); --gpus %d is not supported" % args.gpus)
    import numpy as np
    import torch
    from dldt_amd import builders
    assert torch.cuda.is_available(), "bench.py needs a GPU"

    g, meta = builders.resnet50(batch=args.batch, res=224)
    plan = g.compile(0)
    gen = torch.Generator(device="cuda").manual_seed(20211)

    def run(nreq, steps, warmup):
        """steps inferences round-robin over nreq requests; (ms per step by HIP events, wall ms per step)"""
        reqs = [plan.create_request(perf_count=False) for _ in range(nreq)]
        bufs = [r.device_buffers() for r in reqs]
        for ins, _ in bufs:
            ins[0].copy_(torch.rand(ins[0].shape, generator=gen, device="cuda"))
        streams = [torch.cuda.ExternalStream(r.stream) for r in reqs]
        torch.cuda.synchronize()
        for i in range(warmup):
            reqs[i % nreq].enqueue(*bufs[i % nreq])
        for st in streams:
            st.synchronize()
        torch.cuda.synchronize()
        e0 = [torch.cuda.Event(enable_timing=True) for _ in reqs]
        e1 = [torch.cuda.Event(enable_timing=True) for _ in reqs]
        t0 = time.perf_counter()
        for ev, st in zip(e0, streams):
            ev.record(st)
        for i in range(steps):
            reqs[i % nreq].enqueue(*bufs[i % nreq])
        for ev, st in zip(e1, streams):
            ev.record(st)
        for st in streams:
            st.synchronize()
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) * 1e3
        # the streams start together; the job ends when the last one does
        span = max(a.elapsed_time(b) for a in e0 for b in e1)
        return span / steps, wall / steps, bufs

    ms_per_step, wall_ms_step, bufs = run(args.requests, args.steps, args.warmup)
    wall_ms = wall_ms_step * args.steps
    images_per_s = args.batch / (ms_per_step * 1e-3)
    if args.requests == 1:
        single_ms = ms_per_step
    else:
        single_ms, _, _ = run(1, max(5, min(args.steps, 30)), max(2, args.warmup))
    ins, outs = bufs[0]

    # per-step HIP events on the same stream: time spent in the int8 MFMA kernel
    preq = plan.create_request(perf_count=True)
    acc = {}
    reps = max(3, min(10, args.steps))
    for _ in range(2):
        preq.infer_device(ins, outs)
    for _ in range(reps):
        preq.infer_device(ins, outs)
        for i, st in enumerate(preq.perf()):
            acc[i] = acc.get(i, 0.0) + st["ms"]
    # An event between two kernels costs the stream about 2.7 us (the next dispatch waits for the event's
    # signal): measured here with a small kernel launched back to back and then with an event in front of
    # every launch, and taken off every step, so that a step's time is its kernel's duration (what a
    # kernel trace of the same run shows).
    pstream = torch.cuda.ExternalStream(preq.stream)
    probe = torch.zeros(1 << 20, device="cuda")
    with torch.cuda.stream(pstream):
        n_probe = 50
        for _ in range(5):
            probe.add_(1)
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record(pstream)
        for _ in range(n_probe):
            probe.add_(1)
        b.record(pstream)
        evs = [torch.cuda.Event(enable_timing=True) for _ in range(n_probe + 1)]
        for e in evs[:-1]:
            e.record(pstream)
            probe.add_(1)
        evs[-1].record(pstream)
        pstream.synchronize()
        event_overhead_ms = max(0.0, (evs[0].elapsed_time(evs[-1]) - a.elapsed_time(b)) / n_probe)
    steps = [dict(st, ms=max(acc[i] / reps - event_overhead_ms, 0.0)) for i, st in enumerate(plan.steps)]
    mfma = [s for s in steps if s["type"] in ("Convolution", "Convolution+Shortcut", "MatMul")]
    mfma_ms = sum(s["ms"] for s in mfma)
    mfma_ops = 2.0 * sum(s["macs"] for s in mfma)
    achieved_tops = mfma_ops / (mfma_ms * 1e-3) / 1e12
    total_ops = 2.0 * meta["macs_per_image"] * args.batch

    line = {
        "metric": "ResNet-50 INT8 images/sec @b%d on 1 MI355X" % args.batch,
        "value": images_per_s, "unit": "images/sec", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "u8 x i8 -> i32 (f32 epilogue)", "data": "synthetic",
        "config": {"workload": "ResNet-50 v1.5 INT8 (post-LPT graph), batch %d, 224x224, He-normal weights, "
                               "seeded calibration" % args.batch,
                   "batch": args.batch, "kernels_per_step": len(steps), "wall_ms_per_step": wall_ms / args.steps,
                   "requests_in_flight": args.requests},
        "single_request": {"images_per_sec": args.batch / (single_ms * 1e-3), "ms_per_step": single_ms},
        "tops": total_ops / (ms_per_step * 1e-3) / 1e12,
        "frac_int8_peak_whole_net": total_ops / (ms_per_step * 1e-3) / 1e12 / INT8_PEAK_TOPS,
        "roofline": {"bound": "mfma", "achieved": achieved_tops, "peak": INT8_PEAK_TOPS, "unit": "TFLOP/s",
                     "frac": achieved_tops / INT8_PEAK_TOPS,
                     "traffic": MEASURED_TRAFFIC_BYTES_PER_LAUNCH_B64 if args.batch == 64 else None,
                     "algorithmic_bytes_per_launch": sum(s["bytes"] for s in mfma) / len(mfma),
                     "kernel": "conv_tiled_kernel / conv_pipe_kernel / conv_stream_kernel (all %d convolution/FC launches of one step)" % len(mfma),
                     "ops_per_step": mfma_ops, "kernel_ms_per_step": mfma_ms,
                     "avg_launch_us": mfma_ms * 1e3 / len(mfma), "event_overhead_us": event_overhead_ms * 1e3,
                     "note": "int8 TOP/s, dense peak 5.0 POP/s; launch durations by HIP events around every step on "
                             "the request's stream, less the measured cost of an event between two kernels"},
        "other_kernels_ms_per_step": {t: sum(s["ms"] for s in steps if s["type"] == t)
                                      for t in sorted({s["type"] for s in steps} - {"Convolution", "Convolution+Shortcut", "MatMul"})},
    }
    if not args.no_cpu_baseline:
        line["cpu_baseline"], x_one, want_one = cpu_baseline(args.batch)
        line["parity"] = parity_check(plan, args.batch, x_one, want_one)
        if not line["parity"]["bit_exact"]:
            sys.stderr.write("bench.py: logits differ from the oracle's: %r\n" % (line["parity"],))
    print(json.dumps(line))


if __name__ == "__main__":
    main()
