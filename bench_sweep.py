#!/usr/bin/env python3
"""Sweep of the sampling call over the reference's benchmark grid, beside a plain PyTorch baseline.

The reference's bench.py:32-35 sweeps B in {1..512}, V in {256, 32768, 50304, 65536, 100256,
131072, 151936, 262144}, top_p in {0.1, 0.3, 0.7, 0.9, 1}, top_k in {-1, 1, 10, 100, 1000, 10000}
and five logit generators (bench.py:66-72) against FlashInfer, timing call + synchronize
(bench.py:84-92).  FlashInfer does not exist here; the baseline beside each point is the usual
PyTorch formulation on the same GPU (softmax, descending sort, cumsum, top-k / top-p mask,
multinomial), timed the same way.

    python bench_sweep.py                 # a cross-section of the grid, about a minute
    python bench_sweep.py --full          # the reference's whole grid (11500 points, ten minutes)
    python bench_sweep.py --out sweep.jsonl
    python bench_sweep.py --json results.json --cpu-baseline
    python bench_sweep.py --summarize sweep.jsonl --summary-md summary.md     # no GPU: tables from a finished run

One JSON line per point: shape, parameters, logit generator, microseconds per call for both
(median of call + synchronize, and back-to-back device time between two events), speed-up.
A summary line with the geometric-mean speed-up and the slowest points ends the run.
--json writes one file in the layout of the reference's result file (bench.py:98-138:
benchmark_config / results / summary, times in seconds, medians of call + synchronize), with
`median_torch_gpu_time` in the place of `median_flashinfer_time`; --cpu-baseline adds
`median_torch_cpu_time` (the same PyTorch formulation on the host's cores, timed once per shape and
logit generator: its time does not depend on top_k or top_p) for points of up to 2^21 logits.
Every point starts from a clean routing state (reset_routing): on one stream the library remembers
which kernel suited the last calls, and a sweep changes workload every few calls.
--summary-md writes the tables a reader wants from such a run: per (B, V) the geometric mean and the
minimum of the speed-up and the median time per call, the points furthest from "4 TB/s plus a
launch", the lowest speed-ups, and the CPU column.
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
    for _ in range(3):
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


def geomean(xs):
    return math.exp(sum(math.log(x) for x in xs) / len(xs)) if xs else float("nan")


def distance(r):
    """Back-to-back time over what 4 TB/s plus a 10 us launch would take for the point's logits."""
    return r["us_back_to_back"] / (10.0 + r["B"] * r["V"] * 4 / 4.0e6)


def write_summary_md(path, rows, command):
    """Tables of a finished sweep, as markdown."""
    Bs = sorted({r["B"] for r in rows})
    Vs = sorted({r["V"] for r in rows})
    cell = {}
    for r in rows:
        cell.setdefault((r["B"], r["V"]), []).append(r)
    out = ["# Sweep of the sampling call over the reference's benchmark grid", "",
           "    " + command, "",
           "%d points: B x V x top_p x top_k x logit generator as in the reference's bench.py:32-35, 66-72; "
           "temperature 1.0.  Each point from a clean routing state, 3 untimed calls, then the median of call + "
           "synchronize and the device time of back-to-back calls between two events.  Baseline: the usual PyTorch "
           "formulation (softmax, sort, cumsum, mask, multinomial) on the same GPU, timed the same way "
           "(FlashInfer, the reference's baseline, does not exist here)." % len(rows), "",
           "Over all points: geometric mean of the back-to-back speed-up %.2f (minimum %.2f); of call + synchronize "
           "%.2f (minimum %.2f)." % (geomean([r["speedup_back_to_back"] for r in rows]),
                                      min(r["speedup_back_to_back"] for r in rows),
                                      geomean([r["speedup_call_sync"] for r in rows]),
                                      min(r["speedup_call_sync"] for r in rows)), ""]

    def table(title, fn):
        out.extend(["## " + title, "", "| B \\ V | " + " | ".join(str(v) for v in Vs) + " |",
                    "|---|" + "---|" * len(Vs)])
        for B in Bs:
            out.append("| %d | " % B + " | ".join(fn(cell[(B, V)]) if (B, V) in cell else "" for V in Vs) + " |")
        out.append("")

    table("Speed-up over PyTorch on the GPU, back-to-back: geometric mean (minimum)",
          lambda rs: "%.1f (%.1f)" % (geomean([r["speedup_back_to_back"] for r in rs]),
                                      min(r["speedup_back_to_back"] for r in rs)))
    table("Microseconds per call, back-to-back: median (maximum)",
          lambda rs: "%.1f (%.1f)" % (statistics.median([r["us_back_to_back"] for r in rs]),
                                      max(r["us_back_to_back"] for r in rs)))
    table("Microseconds per call + synchronize: median",
          lambda rs: "%.1f" % statistics.median([r["us_call_sync"] for r in rs]))
    if any("torch_cpu_us" in r for r in rows):
        table("PyTorch on the host CPU (%s threads), microseconds per call: median; ratio to this library's call + synchronize"
              % next(r["torch_cpu_threads"] for r in rows if "torch_cpu_us" in r),
              lambda rs: ("%.0f; %.0fx" % (statistics.median([r["torch_cpu_us"] for r in rs if "torch_cpu_us" in r]),
                                           geomean([r["torch_cpu_us"] / r["us_call_sync"] for r in rs if "torch_cpu_us" in r])))
              if any("torch_cpu_us" in r for r in rs) else "-")

    def listing(title, picked):
        out.extend(["## " + title, "", "| B | V | top_p | top_k | logits | us back-to-back | us call+sync | PyTorch-GPU us | speed-up | x (4 TB/s + 10 us) |",
                    "|---|---|---|---|---|---|---|---|---|---|"])
        for r in picked:
            out.append("| %d | %d | %s | %d | %d | %.1f | %.1f | %.1f | %.2f | %.2f |" % (
                r["B"], r["V"], r["top_p"], r["top_k"], r["logits"], r["us_back_to_back"], r["us_call_sync"],
                r["torch_us_back_to_back"], r["speedup_back_to_back"], distance(r)))
        out.append("")

    listing("Furthest from 4 TB/s plus a launch (back-to-back time over 10 us + bytes / 4 TB/s)",
            sorted(rows, key=lambda r: -distance(r))[:5])
    listing("Lowest speed-ups", sorted(rows, key=lambda r: r["speedup_back_to_back"])[:5])
    out.append("Logit generators (reference bench.py:66-72): 0 zeros, 1 U[0,1), 2 N(0,1)/2, 3 N(0,1)*3, 4 U[0,1)*4.")
    with open(path, "w") as f:
        f.write("\n".join(out) + "\n")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--full", action="store_true", help="the reference's whole grid")
    ap.add_argument("--out", default=None, help="write the JSON lines here as well")
    ap.add_argument("--reps", type=int, default=5, help="timed call+sync repetitions per point (reference: 5)")
    ap.add_argument("--b2b", type=int, default=20, help="back-to-back calls between two events")
    ap.add_argument("--json", default=None, help="write a result file in the reference's layout (bench.py:121-138)")
    ap.add_argument("--cpu-baseline", action="store_true", help="time the PyTorch formulation on the CPU too (small points)")
    ap.add_argument("--summary-md", default=None, help="write the summary tables here as markdown")
    ap.add_argument("--summarize", default=None, help="no run: read the JSON lines of a finished one (--out) and write --summary-md")
    args = ap.parse_args()
    command = "python " + " ".join([os.path.basename(sys.argv[0])] + sys.argv[1:])
    if args.summarize:
        with open(args.summarize) as f:
            recs = [json.loads(l) for l in f if l.strip()]
        command = next((r["command"] for r in recs if "command" in r), command)
        write_summary_md(args.summary_md, [r for r in recs if "B" in r], command)
        return

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
    if out:
        out.write(json.dumps({"command": command}) + "\n")
    speedups, rows = [], []
    n = 0
    for V in Vs:
        for B in Bs:
            states = sample.setup_rand(0, B)
            for kind in kinds:
                logits = make_logits(torch, kind, B, V, gen)
                cpu_us = None
                if args.cpu_baseline and B * V <= (1 << 21):
                    lc = logits.cpu()
                    torch_baseline(torch, lc, 1.0, ks[0], ps[0])
                    ts = []
                    for _ in range(2):
                        t0 = time.perf_counter()
                        torch_baseline(torch, lc, 1.0, ks[0], ps[0])
                        ts.append((time.perf_counter() - t0) * 1e6)
                    cpu_us = statistics.median(ts)
                for top_p in ps:
                    for top_k in ks:
                        if top_k > V:
                            continue
                        ours = lambda: sample.batch_sampling_temperature_topk_topp(logits, states, 1.0, top_k, top_p)
                        base = lambda: torch_baseline(torch, logits, 1.0, top_k, top_p)
                        sample.reset_routing()
                        o_sync, o_b2b = time_call(torch, ours, args.reps, args.b2b)
                        t_sync, t_b2b = time_call(torch, base, args.reps, max(2, args.b2b // 4))
                        rec = {"B": B, "V": V, "top_p": top_p, "top_k": top_k, "logits": kind,
                               "us_call_sync": round(o_sync, 1), "us_back_to_back": round(o_b2b, 1),
                               "torch_us_call_sync": round(t_sync, 1), "torch_us_back_to_back": round(t_b2b, 1),
                               "speedup_call_sync": round(t_sync / o_sync, 2),
                               "speedup_back_to_back": round(t_b2b / o_b2b, 2),
                               "GBps": round(B * V * 4 / o_b2b / 1e3, 1)}
                        if cpu_us is not None:
                            rec["torch_cpu_us"] = round(cpu_us, 1)
                            rec["torch_cpu_threads"] = torch.get_num_threads()
                        line = json.dumps(rec)
                        print(line, flush=True)
                        if out:
                            out.write(line + "\n")
                        speedups.append(t_b2b / o_b2b)
                        rows.append(rec)
                        n += 1
    worst = sorted(rows, key=lambda r: r["speedup_back_to_back"])[:5]
    slow = sorted(rows, key=lambda r: -distance(r))[:5]
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
    if args.summary_md:
        write_summary_md(args.summary_md, rows, command)
    if args.json:
        results = []
        for r in rows:
            e = {"batch_size": r["B"], "vocab_size": r["V"], "top_p": r["top_p"], "top_k": r["top_k"],
                 "logit_type": r["logits"],
                 "median_torch_gpu_time": r["torch_us_call_sync"] * 1e-6,
                 "median_my_kernel_time": r["us_call_sync"] * 1e-6,
                 "speedup_ratio": r["torch_us_call_sync"] / r["us_call_sync"]}
            if "torch_cpu_us" in r:
                e["median_torch_cpu_time"] = r["torch_cpu_us"] * 1e-6
            results.append(e)
        with open(args.json, "w") as f:
            json.dump({"benchmark_config": {"batch_sizes": Bs, "vocab_sizes": Vs, "top_ps": ps, "top_ks": ks,
                                            "logit_types": kinds, "runs_per_setting": args.reps, "temperature": 1.0},
                       "results": results,
                       "summary": {"total_combinations": len(results),
                                   "fastest_kernel_count": {
                                       "torch_gpu": sum(1 for r in results if r["speedup_ratio"] < 1.0),
                                       "your_kernel": sum(1 for r in results if r["speedup_ratio"] >= 1.0)}}},
                      f, indent=2)


if __name__ == "__main__":
    main()
