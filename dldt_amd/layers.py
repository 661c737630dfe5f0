#!/usr/bin/env python3
"""Layer by layer: what each kernel of a plan could take at best, beside what it takes.

    python3 -m dldt_amd.layers                       # ResNet-50 INT8 batch 64: markdown table on stdout
    python3 -m dldt_amd.layers --model mobilenet_v2  # MobileNetV2-1.0 INT8 (bert_encoder: the 12-layer encoder, batch 16 x 384)
    python3 -m dldt_amd.layers --steps-json s.json   # ... and the rows as JSON, followed by 20 inferences back to back on
                                                     #     one request, the last kernels the process launches
    python3 -m dldt_amd.layers --join trace.csv s.json   # the same table with the durations of a kernel trace of that run

Three floors per step, each from the step's own counts and the device's published rates:
  matrix   2 x multiply-accumulates / 5.0 POP/s (dense int8)
  vector   results x instructions of the f32 chain behind the accumulator (every f32 operation of the graph is one
           instruction, as the bit-exact result requires) / (256 compute units x 4 SIMDs x 16 lanes x 2.4 GHz)
  memory   the bytes the step must read and write once (input, weights, residual, output) / 8 TB/s
The attainable time is the largest of the three (all overlapped perfectly); the fraction is attainable / measured.
"""
import argparse
import csv
import json
import sys

INT8_PEAK_OPS = 5.0e15
VALU_LANE_OPS = 256 * 4 * 16 * 2.4e9
HBM_BYTES = 8.0e12
TRACE_TAIL = 20


def floors(step):
    """{'mfma_us', 'valu_us', 'hbm_us', 'attainable_us', 'bound'} of a step dict with macs, bytes, valu_ops"""
    f = {"mfma_us": 2.0 * step["macs"] / INT8_PEAK_OPS * 1e6,
         "valu_us": step.get("valu_ops", 0) / VALU_LANE_OPS * 1e6,
         "hbm_us": step["bytes"] / HBM_BYTES * 1e6}
    bound = max(f, key=f.get)
    f["attainable_us"] = f[bound]
    f["bound"] = bound[:-3]
    return f


def event_overhead_ms(stream_handle):
    """what an event between two kernels costs the stream (the next dispatch waits for the event's signal): a small
    kernel launched back to back, then with an event in front of every launch"""
    import torch
    pstream = torch.cuda.ExternalStream(stream_handle)
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
        return max(0.0, (evs[0].elapsed_time(evs[-1]) - a.elapsed_time(b)) / n_probe)


def step_times(plan, ins, outs, reps=10):
    """the plan's steps with 'ms' (HIP events around every step on one request's stream, less the cost of the event
    itself, so that a step's time is its kernels' duration), 'kernels' and 'valu_ops'; and the event cost in ms"""
    preq = plan.create_request(perf_count=True)
    acc = {}
    for _ in range(2):
        preq.infer_device(ins, outs)
    for _ in range(reps):
        preq.infer_device(ins, outs)
        for i, st in enumerate(preq.perf()):
            acc[i] = acc.get(i, 0.0) + st["ms"]
    over = event_overhead_ms(preq.stream)
    steps = [dict(st, ms=max(acc[i] / reps - over, 0.0), kernels=int(plan.step_rt_info(i, "kernels")),
                  valu_ops=int(plan.step_rt_info(i, "valuOps")))
             for i, st in enumerate(plan.steps)]
    return steps, over


def attainable(steps):
    """{'attainable_ms', 'measured_ms', 'frac', 'bounds'}: sum of the steps' attainable times over the sum of their
    measured ones; bounds counts the steps by the floor that binds them"""
    at = sum(floors(s)["attainable_us"] for s in steps) * 1e-3
    ms = sum(s["ms"] for s in steps)
    bounds = {}
    for s in steps:
        b = floors(s)["bound"]
        bounds[b] = bounds.get(b, 0) + 1
    return {"attainable_ms": at, "measured_ms": ms, "frac": at / ms if ms > 0 else 0.0, "bounds": bounds}


def table(steps, column="ms", label="HIP events"):
    out = ["| # | step | type | variant | GOP | MB | matrix µs | vector µs | memory µs | attainable µs (bound) | measured µs (%s) | attainable / measured |" % label,
           "|---|---|---|---|---|---|---|---|---|---|---|---|"]
    tot_at = tot_ms = 0.0
    for i, s in enumerate(steps):
        f = floors(s)
        us = s[column] * 1e3
        tot_at += f["attainable_us"]
        tot_ms += us
        out.append("| %d | %s | %s | %s | %.2f | %.2f | %.2f | %.2f | %.2f | %.2f (%s) | %.1f | %.2f |" % (
            i, s["name"][-44:], s["type"], s.get("variant", ""), 2e-9 * s["macs"], s["bytes"] / 1e6, f["mfma_us"], f["valu_us"],
            f["hbm_us"], f["attainable_us"], f["bound"], us, f["attainable_us"] / us if us > 0 else 0.0))
    out.append("| | **all %d steps** | | | %.1f | %.1f | %.1f | %.1f | %.1f | %.1f | %.1f | **%.3f** |" % (
        len(steps), sum(2e-9 * s["macs"] for s in steps), sum(s["bytes"] for s in steps) / 1e6,
        sum(floors(s)["mfma_us"] for s in steps), sum(floors(s)["valu_us"] for s in steps),
        sum(floors(s)["hbm_us"] for s in steps), tot_at, tot_ms, tot_at / tot_ms if tot_ms > 0 else 0.0))
    return "\n".join(out)


def join(trace_csv, steps_json):
    """the steps with 'trace_ms': the kernel trace's durations of the last TRACE_TAIL inferences, averaged step by step"""
    with open(steps_json) as f:
        steps = json.load(f)
    rows = []
    with open(trace_csv, newline="") as f:
        for r in csv.DictReader(f):
            rows.append((int(r["Start_Timestamp"]), int(r["End_Timestamp"]), r["Kernel_Name"]))
    rows.sort()
    per = sum(s["kernels"] for s in steps)
    tail = rows[-per * TRACE_TAIL:]
    assert len(tail) == per * TRACE_TAIL, "the trace holds %d kernels, %d expected at least" % (len(rows), per * TRACE_TAIL)
    names = [r[2] for r in tail]
    for k in range(1, TRACE_TAIL):          # the same kernels in the same order, inference after inference
        assert names[k * per:(k + 1) * per] == names[:per], "inference %d of the trace's tail launches other kernels" % k
    at = 0
    for s in steps:
        ns = 0
        for k in range(TRACE_TAIL):
            for j in range(s["kernels"]):
                a, b, _ = tail[k * per + at + j]
                ns += b - a
        s["trace_ms"] = ns / TRACE_TAIL * 1e-6
        s["trace_kernels"] = ", ".join(sorted({n.split("(")[0][-60:] for n in names[at:at + s["kernels"]]}))
        at += s["kernels"]
    return steps


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--model", choices=("resnet50", "mobilenet_v2", "bert_encoder"), default="resnet50")
    ap.add_argument("--tune-streams", type=int, default=0, help="requests the kernels are chosen for at load (0: the library's default)")
    ap.add_argument("--steps-json")
    ap.add_argument("--join", nargs=2, metavar=("TRACE_CSV", "STEPS_JSON"))
    args = ap.parse_args()
    if args.join:
        steps = join(*args.join)
        print(table(steps, "trace_ms", "kernel trace"))
        a = attainable([dict(s, ms=s["trace_ms"]) for s in steps])
        print("\nattainable %.3f ms, traced %.3f ms: fraction %.3f; steps by binding floor: %s" % (
            a["attainable_ms"], a["measured_ms"], a["frac"], a["bounds"]))
        return
    import torch
    from . import builders
    assert torch.cuda.is_available(), "needs a GPU"
    if args.model == "bert_encoder":     # 12 layers, hidden 768, sequence 384; --batch 64 stands for its own batch of 16
        g, _ = builders.bert_encoder(batch=16 if args.batch == 64 else args.batch)
    else:
        g, _ = (builders.resnet50 if args.model == "resnet50" else builders.mobilenet_v2)(batch=args.batch, res=224)
    plan = g.compile(0, config={"HIP_THROUGHPUT_STREAMS": str(args.tune_streams)} if args.tune_streams else None)
    req = plan.create_request()
    ins, outs = req.device_buffers()
    for t in ins:
        t.copy_(torch.rand(t.shape, device="cuda") if t.dtype == torch.float32 else torch.zeros(t.shape, device="cuda").to(t.dtype))
    torch.cuda.synchronize()
    steps, over = step_times(plan, ins, outs)
    print(table(steps))
    a = attainable(steps)
    print("\nattainable %.3f ms, measured %.3f ms: fraction %.3f; steps by binding floor: %s; an event costs %.1f µs" % (
        a["attainable_ms"], a["measured_ms"], a["frac"], a["bounds"], over * 1e3))
    sys.stdout.flush()
    if args.steps_json:
        with open(args.steps_json, "w") as f:
            json.dump(steps, f)
        stream = torch.cuda.ExternalStream(req.stream)
        torch.cuda.synchronize()
        for _ in range(TRACE_TAIL):
            req.enqueue(ins, outs)
        stream.synchronize()


if __name__ == "__main__":
    main()
