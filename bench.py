#!/usr/bin/env python3
"""Benchmark of the sampling hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload of the headline number (BASELINE.json configs[1]): B=1, V=262144,
logits N(0,1)*3 (seeded, synthetic), temperature 1.0, top_k -1, top_p 0.3; a
"step" is one call of batch_sampling_temperature_topk_topp through the drop-in
Python module with the logits already resident in HBM.  `value` is the median
device-side time of one call in microseconds (HIP events around each call on the
stream the kernel runs on).  Next to it, in the same JSON line:

  latency    the launch-plus-one-read floor kernel timed the same way, the
             ratio to it, the wall-clock "call + synchronize" time the
             reference's own bench measures (reference bench.py:84-92) for the
             call and for the floor kernel (what a launch and a synchronize
             cost on this host whatever the kernel does), and
             `readme_point`: the one point the reference publishes
             (README.md:21-31: same shape, logits U[0,1)*4)
  roofline   the bandwidth-bound configuration (BASELINE.json configs[4]):
             logits (128,4,1048576) fp32 = 2 GiB resident, top_k 1024,
             top_p 0.95; algorithmic bytes = 4*V per sampled row; the time
             is that of the whole call (its two launches), averaged over
             back-to-back calls between two HIP events; beside it the same
             rows with penalties (12*V algorithmic bytes per row)
  configs    time per call and rows/s of the other BASELINE configurations
  cpu_baseline  the CPU oracle (single thread) on a bounded sample of the
             headline workload; cpu_torch is torch-CPU softmax/sort/cumsum/
             multinomial on the same row with its thread count
"""
import argparse
import json
import os
import statistics
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0   # MI355X HBM3E, vendor figure

# HBM bytes per call of the bandwidth configuration from the rocprofv3 FETCH_SIZE / WRITE_SIZE runs
# summarised in the file named here, valid for the library version they were taken with: a library
# that has moved on reports traffic as null rather than a stale figure.
TRAFFIC_PROFILE = {"file": "profiles/bench_kernels_hbm_traffic_pmc.md", "rs_version": 415, "bytes": 573847962}


def event_times_us(torch, fn, steps, warmup):
    """Median / mean device time of fn() in microseconds, from one event pair per call
    recorded on the current stream, plus the wall-clock time of the whole timed region."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        starts[i].record()
        fn()
        ends[i].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    us = [s.elapsed_time(e) * 1000.0 for s, e in zip(starts, ends)]
    return us, wall


def block_time_us(torch, fn, steps, warmup):
    """Average device time per call over `steps` back-to-back calls (one event pair around all)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(steps):
        fn()
    e.record()
    torch.cuda.synchronize()
    return s.elapsed_time(e) * 1000.0 / steps


def sync_call_us(torch, fn, reps):
    """Wall clock of call + synchronize, as the reference's bench takes it."""
    out = []
    for _ in range(reps):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        out.append((time.perf_counter() - t0) * 1e6)
    return out


def pct(xs, q):
    xs = sorted(xs)
    return xs[min(len(xs) - 1, int(q * len(xs)))]


def cpu_baselines(logits_row_np, temperature, top_k, top_p, budget_s=12.0):
    """Oracle (port, 1 thread) and torch-CPU sort/cumsum/multinomial on the headline row."""
    import numpy as np
    import torch
    from oracle import oracle as O

    V = logits_row_np.shape[0]
    c, k, p = O.normalize(temperature, top_k, top_p, V)
    O.sample_row(logits_row_np, c, k, p, u=0.5)
    n, t0 = 0, time.perf_counter()
    while time.perf_counter() - t0 < budget_s:
        O.sample_row(logits_row_np, c, k, p, u=0.25 + 0.5 * ((n * 0.618) % 1.0))
        n += 1
    oracle_us = (time.perf_counter() - t0) / n * 1e6
    port = {"value": round(oracle_us, 1), "unit": "us/call", "cores": 1, "kind": "port",
            "sample": "%d calls of the oracle on the same B=1, V=%d row (%.0f s)" % (n, V, budget_s)}

    x = torch.from_numpy(logits_row_np)[None, :]
    kk = V if top_k <= 0 or top_k > V else top_k

    def torch_cpu():
        probs = torch.softmax(x / temperature, dim=-1)
        sp, si = torch.sort(probs, dim=-1, descending=True)
        cs = torch.cumsum(sp, dim=-1)
        keep = (cs - sp < top_p) & (torch.arange(V)[None, :] < kk)
        w = torch.where(keep, sp, torch.zeros_like(sp))
        j = torch.multinomial(w, 1)
        return si.gather(-1, j)

    torch_cpu()
    m, t0 = 0, time.perf_counter()
    while time.perf_counter() - t0 < budget_s / 2:
        torch_cpu()
        m += 1
    tus = (time.perf_counter() - t0) / m * 1e6
    tc = {"value": round(tus, 1), "unit": "us/call", "cores": torch.get_num_threads(),
          "host_cpus": os.cpu_count(), "kind": "torch-cpu softmax/sort/cumsum/multinomial",
          "sample": "%d calls on the same row" % m}
    return port, tc


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--skip-bandwidth", action="store_true", help="skip the 2 GiB bandwidth configuration")
    ap.add_argument("--skip-cpu", action="store_true", help="skip the CPU baselines")
    ap.add_argument("--bandwidth-steps", type=int, default=20)
    ap.add_argument("--traffic-probe", action="store_true",
                    help="also run one plain device copy of 512 MiB (read 512 MiB + write 512 MiB), the known-size "
                         "kernel that rocprofv3 FETCH_SIZE / WRITE_SIZE readings are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (rows shard over GPUs without communication; "
              "no multi-GPU path is part of it). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    import rapid_sampling_amd as sample

    import ctypes
    lib_version = ctypes.CDLL(sample.KERNEL_LIBRARY).rs_version()
    assert torch.cuda.is_available(), "bench.py needs the GPU"
    torch.cuda.set_device(0)
    dev = torch.device("cuda:0")

    # ---- headline: B=1, V=262144 -------------------------------------------
    V, temperature, top_k, top_p = 262144, 1.0, -1, 0.3
    row_np = (np.random.default_rng(1).standard_normal(V, dtype=np.float32) * np.float32(3.0)).astype(np.float32)
    logits = torch.from_numpy(row_np)[None, :].to(dev)
    states = sample.setup_rand(0, 1)

    def call():
        return sample.batch_sampling_temperature_topk_topp(logits, states, temperature, top_k, top_p)

    def floor():
        return sample.floor_read(logits)

    us, wall = event_times_us(torch, call, args.steps, args.warmup)
    p50 = statistics.median(us)
    floor_us, _ = event_times_us(torch, floor, min(args.steps, 2000), min(args.warmup, 100))
    floor_p50 = statistics.median(floor_us)
    sync_us = sync_call_us(torch, call, 200)
    floor_sync_us = sync_call_us(torch, floor, 200)
    b2b_us = block_time_us(torch, call, min(args.steps, 2000), 20)
    floor_b2b_us = block_time_us(torch, floor, min(args.steps, 2000), 20)

    # the reference's one published point: same B, V, top_k, top_p, logits U[0,1)*4 (bench.py:72, logit type 4)
    flat_np = (np.random.default_rng(4).random(V, dtype=np.float32) * np.float32(4.0)).astype(np.float32)
    flat = torch.from_numpy(flat_np)[None, :].to(dev)
    side = torch.cuda.Stream()                            # its own stream: its own workspace and routing state

    def call_flat_row():
        return sample.batch_sampling_temperature_topk_topp(flat, states, temperature, top_k, top_p)

    with torch.cuda.stream(side):
        readme_us, _ = event_times_us(torch, call_flat_row, min(args.steps, 2000), min(args.warmup, 100))
        readme_sync = sync_call_us(torch, call_flat_row, 200)
        readme_state = sample._sample.policy_state()
    side.synchronize()
    readme_p50 = statistics.median(readme_us)

    result = {
        "metric": "p50 us/call (B=1,V=256K); HBM GB/s vs peak at B=128x4,V=1M",
        "value": round(p50, 3),
        "unit": "us/call",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall / args.steps * 1e3, 6),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "B=1, V=262144, logits N(0,1)*3 seed 1, temperature 1.0, top_k -1, top_p 0.3, "
                               "Philox draws, drop-in Python call"},
        "latency": {
            "p50_us": round(p50, 3), "p10_us": round(pct(us, 0.10), 3), "p90_us": round(pct(us, 0.90), 3),
            "p99_us": round(pct(us, 0.99), 3), "max_us": round(max(us), 3),
            "back_to_back_us": round(b2b_us, 3),
            "floor_p50_us": round(floor_p50, 3), "floor_back_to_back_us": round(floor_b2b_us, 3),
            "ratio_to_floor": round(p50 / floor_p50, 3),
            "call_plus_sync_p50_us": round(statistics.median(sync_us), 2),
            "floor_call_plus_sync_p50_us": round(statistics.median(floor_sync_us), 2),
            "reference_call_plus_sync_us": 220.3,
            "reference_note": "reference README.md:21-31: same B, V, top_p, top_k, logits U[0,1)*4, unnamed NVIDIA GPU",
            "readme_point": {
                "workload": "B=1, V=262144, logits U[0,1)*4 seed 4, temperature 1.0, top_k -1, top_p 0.3 (README.md:21-31)",
                "p50_us": round(readme_p50, 3), "p99_us": round(pct(readme_us, 0.99), 3), "max_us": round(max(readme_us), 3),
                "ratio_to_floor": round(readme_p50 / floor_p50, 3),
                "call_plus_sync_p50_us": round(statistics.median(readme_sync), 2),
                "path": "general kernel (the flat row's nucleus is too large for the streaming path; routed by its reports)"
                        if readme_state & 1 else "streaming path",
                "reference_call_plus_sync_us": 220.3,
            },
        },
    }

    # ---- bandwidth: (128, 4, 1048576), 2 GiB resident ------------------------
    if not args.skip_bandwidth:
        Bb, Tb, Vb = 128, 4, 1048576
        g = torch.Generator(device=dev)
        g.manual_seed(5)
        big = torch.randn((Bb, Tb, Vb), generator=g, device=dev, dtype=torch.float32)
        big.mul_(1.5)
        st_b = sample.setup_rand(1, Bb * Tb)

        def call_btv():
            return sample.batch_sampling_temperature_topk_topp(big, st_b, 1.0, 1024, 0.95)

        flat = big.view(Bb * Tb, Vb)

        def call_flat():
            return sample.batch_sampling_temperature_topk_topp(flat, st_b, 1.0, 1024, 0.95)

        def floor_variant(n):
            return lambda: sample.floor_read(big, n)

        t_btv = block_time_us(torch, call_btv, args.bandwidth_steps, 3)
        t_flat = block_time_us(torch, call_flat, max(2, args.bandwidth_steps // 2), 2)
        # read-only kernels on the same rows: plain / non-temporal loads on the general kernel's grid
        # and on the streaming pass's grid
        floor_names = ["plain loads, 128 KiB per workgroup", "non-temporal loads, 128 KiB per workgroup",
                       "plain loads, 64 KiB per workgroup", "non-temporal loads, 64 KiB per workgroup",
                       "persistent grid of 2048 workgroups, 4 loads in flight", "the same, an eighth of the data per XCD",
                       "256 KiB contiguous per workgroup, 16 loads in flight",
                       "persistent grid of 1024 workgroups, an eighth of the data per XCD, 8 loads in flight",
                       "persistent grid of 4096 workgroups, 2 loads in flight"]
        t_floors = [block_time_us(torch, floor_variant(n), args.bandwidth_steps, 3) for n in range(len(floor_names))]
        t_floor = min(t_floors)
        sample._sample.force_path("cluster")             # the general single-launch kernel on the same input
        try:
            t_cluster = block_time_us(torch, call_btv, max(2, args.bandwidth_steps // 2), 2)
        finally:
            sample._sample.force_path("auto")
        bytes_btv = Bb * Vb * 4
        bytes_flat = Bb * Tb * Vb * 4
        ach = bytes_btv / (t_btv * 1e-6) / 1e9
        result["roofline"] = {
            "bound": "hbm", "achieved": round(ach, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(ach / HBM_PEAK_GBS, 4),
            "traffic": TRAFFIC_PROFILE["bytes"] if lib_version == TRAFFIC_PROFILE["rs_version"] else None,
            "traffic_source": "%s (library version %d; running %d)" % (TRAFFIC_PROFILE["file"], TRAFFIC_PROFILE["rs_version"], lib_version),
            "workload": "(B,T,V)=(128,4,1048576) N(0,1.5), top_k 1024, top_p 0.95: 128 sampled rows of 4 MiB, "
                        "stride T*V, algorithmic bytes 4*V per row = 512 MiB per call",
            "us_per_call": round(t_btv, 2), "rows_per_s": round(Bb / (t_btv * 1e-6), 1),
            "kernels": "streaming path, two launches per call: rs::stream_kernel (reads the logits; dominant) and "
                       "rs::finish_kernel; achieved = bytes / time of the whole call",
            "cluster_path_us_per_call": round(t_cluster, 2),
            "read_peak_GBs": round(bytes_btv / (t_floor * 1e-6) / 1e9, 1),
            "frac_of_read_peak": round(t_floor / t_btv, 4),
            "read_only_kernels_GBs": {n: round(bytes_btv / (t * 1e-6) / 1e9, 1) for n, t in zip(floor_names, t_floors)},
            "flattened_512_rows": {"us_per_call": round(t_flat, 2),
                                   "achieved": round(bytes_flat / (t_flat * 1e-6) / 1e9, 1),
                                   "rows_per_s": round(Bb * Tb / (t_flat * 1e-6), 1)},
        }
        # the same rows with plain temperature sampling (top_k = V, top_p = 1: every live token kept)
        def call_plain():
            return sample.batch_sampling_temperature_topk_topp(big, st_b, 1.0, -1, 1.0)

        t_plain = block_time_us(torch, call_plain, args.bandwidth_steps, 3)
        result["roofline"]["plain_temperature"] = {
            "us_per_call": round(t_plain, 2), "achieved": round(bytes_btv / (t_plain * 1e-6) / 1e9, 1),
            "frac": round(bytes_btv / (t_plain * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
            "note": "the same (128,4,1048576) call with top_k -1, top_p 1.0: rs::stream_kernel counts only (no stashes), "
                    "rs::finish_kernel picks the slice from the slices' masses and reads that slice once more"}
        # extension: the same rows handed over as bfloat16 (half the algorithmic bytes); (128, 1M), T = 1
        half = big[:, Tb - 1, :].to(torch.bfloat16)
        st_h = sample.setup_rand(1, Bb)

        def call_half():
            return sample.batch_sampling_temperature_topk_topp(half, st_h, 1.0, 1024, 0.95, accept_half=True)

        t_half = block_time_us(torch, call_half, args.bandwidth_steps, 3)
        result["roofline"]["bfloat16_logits_extension"] = {
            "us_per_call": round(t_half, 2), "achieved": round(Bb * Vb * 2 / (t_half * 1e-6) / 1e9, 1),
            "note": "(128,1048576) bfloat16 rows of the same values rounded, 2*V bytes per row, accept_half=True"}
        del half
        # the same rows with penalties: logits and penalties read once, penalties rewritten once the
        # tokens are known -- 12*V algorithmic bytes per row (4*V logits, 4*V + 4*V penalties)
        pen_b = torch.where(torch.rand((Bb, Vb), generator=g, device=dev) < 0.02,
                            torch.empty((Bb, Vb), device=dev).exponential_(1.0, generator=g),
                            torch.zeros((), device=dev))
        last = big[:, Tb - 1, :]

        def call_pen():
            return sample.batch_sampling_repetition_temperature_topk_topp(last, pen_b, st_h, 0.1, 0.1, 0.95, 1.0, 1024, 0.95)

        t_pen = block_time_us(torch, call_pen, max(2, args.bandwidth_steps // 2), 2)
        result["roofline"]["with_penalties"] = {
            "us_per_call": round(t_pen, 2), "achieved": round(Bb * Vb * 12 / (t_pen * 1e-6) / 1e9, 1),
            "frac": round(Bb * Vb * 12 / (t_pen * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
            "note": "(128,1048576) fp32 rows (stride T*V) with a (128,1048576) penalties tensor, 2 % non-zero: "
                    "rs::stream_pen_kernel (reads both, writes the decayed penalties), rs::finish_kernel (patches the sampled "
                    "tokens), rs::penalty_fix_kernel (slices the pass deferred: none here); algorithmic bytes 12*V per row"}
        del pen_b, last
        # kept sets of thousands of tokens (calls of this size take the one-pass wide path: a look at a sample of
        # each row, one pass over the logits, a finish per row): the same rows with top_k 10000, and 512 flat
        # rows of 262144 tokens with a nucleus of 0.9; beside them the two-pass wide path (counting pass, plan,
        # second pass around the boundary bin, finish) and the general kernel
        def call_wide_k():
            return sample.batch_sampling_temperature_topk_topp(big, st_b, 1.0, 10000, 1.0)

        t_wk = block_time_us(torch, call_wide_k, max(2, args.bandwidth_steps // 2), 3)
        sample._sample.force_path("cluster")
        try:
            t_wk_cluster = block_time_us(torch, call_wide_k, 2, 1)
            sample._sample.force_path("wide")
            t_wk_two = block_time_us(torch, call_wide_k, max(2, args.bandwidth_steps // 2), 2)
        finally:
            sample._sample.force_path("auto")
        flat_rows = torch.rand((512, 262144), generator=g, device=dev)
        st_w = sample.setup_rand(2, 512)

        def call_wide_p():
            return sample.batch_sampling_temperature_topk_topp(flat_rows, st_w, 1.0, -1, 0.9)

        t_wp = block_time_us(torch, call_wide_p, max(2, args.bandwidth_steps // 2), 3)
        sample._sample.force_path("wide")
        try:
            t_wp_two = block_time_us(torch, call_wide_p, max(2, args.bandwidth_steps // 2), 2)
        finally:
            sample._sample.force_path("auto")
        # the same kind of kept set in many short rows: the row kernel (one workgroup per row, the row in registers)
        short_rows = torch.rand((512, 50304), generator=g, device=dev)

        def call_row():
            return sample.batch_sampling_temperature_topk_topp(short_rows, st_w, 1.0, 10000, 1.0)

        t_row = block_time_us(torch, call_row, 20, 3)
        sample._sample.force_path("cluster")
        try:
            t_row_cluster = block_time_us(torch, call_row, 10, 2)
        finally:
            sample._sample.force_path("auto")
        del short_rows
        result["roofline"]["wide_kept_sets"] = {
            "top_k_10000": {"us_per_call": round(t_wk, 2), "achieved": round(bytes_btv / (t_wk * 1e-6) / 1e9, 1),
                            "frac": round(bytes_btv / (t_wk * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
                            "two_pass_us_per_call": round(t_wk_two, 2),
                            "cluster_path_us_per_call": round(t_wk_cluster, 2)},
            "flat_512x262144_top_p_0.9": {"us_per_call": round(t_wp, 2),
                                          "achieved": round(512 * 262144 * 4 / (t_wp * 1e-6) / 1e9, 1),
                                          "frac": round(512 * 262144 * 4 / (t_wp * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
                                          "two_pass_us_per_call": round(t_wp_two, 2)},
            "flat_512x50304_top_k_10000": {"us_per_call": round(t_row, 2),
                                           "achieved": round(512 * 50304 * 4 / (t_row * 1e-6) / 1e9, 1),
                                           "frac": round(512 * 50304 * 4 / (t_row * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
                                           "cluster_path_us_per_call": round(t_row_cluster, 2),
                                           "note": "rs::row_kernel, one launch: a workgroup of 1024 threads per row, two rounds "
                                                   "of 256 rows; bound by its vector instructions, not by the read"},
            "note": "one-pass wide path, three launches: rs::wide_sample_kernel (a sample of each row, 32768 tokens at "
                    "most), rs::wide1_kernel (the pass over the logits), rs::wide1_finish_kernel; two_pass: "
                    "rs::stream_kernel (counting only), rs::wide_plan_kernel, rs::wide_kernel (reads the logits a second "
                    "time), rs::wide_finish_kernel; achieved = algorithmic bytes 4*V per row / time of the whole call"}
        del flat_rows
        if args.traffic_probe:
            src = big.view(-1)[: Bb * Vb]
            dst = torch.empty_like(src)
            dst.copy_(src)
            torch.cuda.synchronize()
            del dst
        del big, flat

    # ---- the other BASELINE configurations (parity cases; time and rows/s only) ----
    def timed_rows(fn, B, steps=200):
        t = block_time_us(torch, fn, steps, 10)
        return {"us_per_call": round(t, 2), "rows_per_s": round(B / (t * 1e-6), 1)}

    g1 = torch.Generator(device=dev)
    g1.manual_seed(0)
    c1 = torch.rand((1, 131072), generator=g1, device=dev)
    st1 = sample.setup_rand(0, 1)
    g3 = torch.Generator(device=dev)
    g3.manual_seed(4)
    c3 = torch.randn((64, 152064), generator=g3, device=dev) * 2.0
    c3.scatter_add_(1, torch.randint(0, 152064, (64, 16), generator=g3, device=dev),
                    torch.full((64, 16), 10.0, device=dev))
    st3 = sample.setup_rand(3, 64)
    g4 = torch.Generator(device=dev)
    g4.manual_seed(40)
    c4 = torch.randn((32, 131072), generator=g4, device=dev) * 1.5
    pen4 = torch.where(torch.rand((32, 131072), generator=g4, device=dev) < 0.02,
                       torch.empty((32, 131072), device=dev).exponential_(1.0, generator=g4),
                       torch.zeros((), device=dev))
    st4 = sample.setup_rand(4, 32)
    result["configs"] = {
        "C1 B=1 V=131072 U[0,1) top_p 0.5": timed_rows(
            lambda: sample.batch_sampling_temperature_topk_topp(c1, st1, 1.0, -1, 0.5), 1),
        "C3 B=64 V=152064 N(0,2)+spikes T 0.8 top_k 50 top_p 0.9": timed_rows(
            lambda: sample.batch_sampling_temperature_topk_topp(c3, st3, 0.8, 50, 0.9), 64),
        "C4 B=32 V=131072 penalties, 256 chained calls on fixed logits": timed_rows(
            lambda: sample.batch_sampling_repetition_temperature_topk_topp(c4, pen4, st4, 0.1, 0.1, 0.95,
                                                                           0.8, 50, 0.9), 32, steps=256),
    }
    del c1, c3, c4, pen4

    # ---- CPU baselines ------------------------------------------------------
    if not args.skip_cpu:
        port, tc = cpu_baselines(row_np, temperature, top_k, top_p)
        result["cpu_baseline"] = port
        result["cpu_torch"] = tc

    print(json.dumps(result))


if __name__ == "__main__":
    main()
