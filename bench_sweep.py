#!/usr/bin/env python3
"""Sweep of the sampling call over the reference's benchmark grid, beside a plain PyTorch baseline.

The reference's bench.py:32-35 sweeps B in {1..512}, V in {256, 32768, 50304, 65536, 100256,
131072, 151936, 262144}, top_p in {0.1, 0.3, 0.7, 0.9, 1}, top_k in {-1, 1, 10, 100, 1000, 10000}
and five logit generators (bench.py:66-72) against FlashInfer, timing call + synchronize
(bench.py:84-92).  FlashInfer does not exist here; the baseline beside each point is the usual
PyTorch formulation on the same GPU (softmax, descending sort, cumsum, top-k / top-p mask,
multinomial), timed the same way.

    python bench_sweep.py                 # a cross-section of the grid, about a minute
    python bench_sweep.py --full          # the reference's whole grid (7200 points)
    python bench_sweep.py --out sweep.jsonl

One JSON line per point: shape, parameters, logit generator, microseconds per call for both
(median of call + synchronize, and back-to-back device time between two events), speed-up.
A summary line with the geometric-mean speed-up and the slowest points ends the run.
"""
import argparse
import json
import math
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def make_logits(torch, kind, B, V, gen):
    """The reference's five generators (bench.py:66-72)."""
    if kind == 0:
        return torch.zeros(B, V, dtype=torch.float32, device="cuda")
    if kind == 1:
        return torch.rand(B, V, dtype=torch.float32, device="cuda", generator=gen)
    if kind == 2:
        return torch.randn(B, V, dtype=torch.float32, device="cuda", generator=gen) / 2
    if kind == 3:
        return torch.randn(B, V, dtype=torch.float32, device="cuda", generator=gen) * 3
    return torch.rand(B, V, dtype=torch.float32, device="cuda", generator=gen) * 4


def torch_baseline(torch, logits, temperature, top_k, top_p):
    V = logits.shape[-1]
    probs = torch.softmax(logits / temperature, dim=-1)
    sp, si = torch.sort(probs, dim=-1, descending=True)
    cs = torch.cumsum(sp, dim=-1)
    keep = cs - sp < top_p
    if 0 < top_k < V:
        keep[..., top_k:] = False
    w = torch.where(keep, sp, torch.zeros((), device=sp.device))
    return si.gather(-1, torch.multinomial(w, 1)).squeeze(-1)


def time_call(torch, fn, reps, b2b):
    fn()
    fn()
    torch.cuda.synchronize()
    ts = []
    for _ in range(reps):
        t0 = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        ts.append((time.perf_counter() - t0) * 1e6)
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(b2b):
        fn()
    e.record()
    torch.cuda.synchronize()
    return statistics.median(ts), s.elapsed_time(e) * 1000.0 / b2b


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--full", action="store_true", help="the reference's whole grid")
    ap.add_argument("--out", default=None, help="write the JSON lines here as well")
    ap.add_argument("--reps", type=int, default=5, help="timed call+sync repetitions per point (reference: 5)")
    ap.add_argument("--b2b", type=int, default=20, help="back-to-back calls between two events")
    args = ap.parse_args()

    import torch

    import rapid_sampling_amd as sample

    assert torch.cuda.is_available(), "bench_sweep.py needs the GPU"
    if args.full:
        Bs = [1, 2, 4, 8, 16, 32, 64, 128, 256, 512]
        Vs = [256, 32768, 50304, 65536, 100256, 131072, 151936, 262144]
        ps = [0.1, 0.3, 0.7, 0.9, 1]
        ks = [-1, 1, 10, 100, 1000, 10000]
        kinds = [0, 1, 2, 3, 4]
    else:
        Bs = [1, 8, 64, 512]
        Vs = [256, 32768, 151936, 262144]
        ps = [0.3, 0.9, 1]
        ks = [-1, 100]
        kinds = [1, 3]
    gen = torch.Generator(device="cuda")
    gen.manual_seed(0)
    out = open(args.out, "w") if args.out else None
    speedups, rows = [], []
    n = 0
    for V in Vs:
        for B in Bs:
            states = sample.setup_rand(0, B)
            for kind in kinds:
                logits = make_logits(torch, kind, B, V, gen)
                for top_p in ps:
                    for top_k in ks:
                        if top_k > V:
                            continue
                        ours = lambda: sample.batch_sampling_temperature_topk_topp(logits, states, 1.0, top_k, top_p)
                        base = lambda: torch_baseline(torch, logits, 1.0, top_k, top_p)
                        o_sync, o_b2b = time_call(torch, ours, args.reps, args.b2b)
                        t_sync, t_b2b = time_call(torch, base, args.reps, max(2, args.b2b // 4))
                        rec = {"B": B, "V": V, "top_p": top_p, "top_k": top_k, "logits": kind,
                               "us_call_sync": round(o_sync, 1), "us_back_to_back": round(o_b2b, 1),
                               "torch_us_call_sync": round(t_sync, 1), "torch_us_back_to_back": round(t_b2b, 1),
                               "speedup_call_sync": round(t_sync / o_sync, 2),
                               "speedup_back_to_back": round(t_b2b / o_b2b, 2),
                               "GBps": round(B * V * 4 / o_b2b / 1e3, 1)}
                        line = json.dumps(rec)
                        print(line, flush=True)
                        if out:
                            out.write(line + "\n")
                        speedups.append(t_b2b / o_b2b)
                        rows.append(rec)
                        n += 1
    worst = sorted(rows, key=lambda r: r["speedup_back_to_back"])[:5]
    slow = sorted(rows, key=lambda r: -r["us_back_to_back"] / max(1.0, r["B"] * r["V"] * 4 / 4.0e6))[:5]
    summary = {"points": n,
               "geomean_speedup_back_to_back": round(math.exp(sum(math.log(x) for x in speedups) / len(speedups)), 2),
               "min_speedup_back_to_back": round(min(speedups), 2),
               "lowest_speedups": worst,
               "furthest_from_4TBps_plus_launch": slow}
    line = json.dumps({"summary": summary})
    print(line, flush=True)
    if out:
        out.write(line + "\n")
        out.close()


if __name__ == "__main__":
    main()
