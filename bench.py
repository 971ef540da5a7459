#!/usr/bin/env python3
"""Benchmark of the row-reduction / elementwise hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg2] [--no-extra] [--no-cpu]

A step is one pass of the hot path over one batch of the headline workload (cfg2: RMSNorm
forward + reverse, r32, [8192, 4096]) with all inputs resident in HBM. Successive steps
rotate over several buffer sets, and the reverse of a step works on a different set than its
forward, so the 256 MiB memory-side cache cannot serve repeats. One JSON line is printed:
whole-step throughput (`value`, GB/s of algorithmic bytes), the roofline of the dominant
launcher measured with events on the launch stream inside the timed region, the CPU oracle
timed on the host cores, and (unless --no-extra) forward/reverse rates of the other workloads.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBPS = 8000.0
SETS = {"cfg1": 16, "cfg2": 4, "cfg3": 2, "cfg4": 2, "cfg5a": 3, "cfg5b": 3, "copy": 2, "permutate": 2, "gemm": 2}
MFMA_PEAK_TFLOPS = {"gemm": 2500.0}  # dense fp16 matrix rate of the MI355X


PROFILE_OF = {"cfg1": "cfg1_softmax", "cfg2": "cfg2_rmsnorm", "cfg3": "cfg3_softmax_r16",
              "cfg4": "cfg4_fused_chain", "cfg5a": "cfg5a_softmax_vocab", "cfg5b": "cfg5b_softmax_vocab",
              "permutate": "permutate_transpose", "gemm": "gemm_rocblas_r16"}


def traffic_from_profile(name):
    """HBM bytes per launch of the dominant launcher, as derived from the rocprofv3 FETCH_SIZE /
    WRITE_SIZE runs summarised under profiles/ (None when no summary is committed)."""
    import re
    path = os.path.join(ROOT, "profiles", f"{PROFILE_OF.get(name, name)}_hbm_traffic.md")
    if not os.path.exists(path):
        return None
    with open(path) as f:
        m = re.search(r"roofline_traffic_bytes_per_launch\s*=\s*(\d+)", f.read())
    return int(m.group(1)) if m else None


def _events(n):
    import torch
    return [torch.cuda.Event(enable_timing=True) for _ in range(n)]


def _median(v):
    s = sorted(v)
    return s[len(s) // 2]


def make_sets(name, count=None):
    from metaphor_amd import workloads as W
    return [W.WORKLOADS[name](seed=i) for i in range(count or SETS[name])]


EVENT_EVERY = 8  # a pair of events costs ~2-5 us of stream time: sample launches, not every one


def time_steps(sets, steps, warmup):
    """K timed steps. Returns (seconds, durations in ms of the dominant launcher sampled with
    events inside the timed region on the launch stream)."""
    import torch
    S = len(sets)
    rev_of = lambda i: sets[(i + S // 2) % S]
    has_rev = sets[0].has_reverse
    for s in sets:  # every set's forward output exists before any reverse consumes it
        s.forward()
    for i in range(warmup):
        sets[i % S].forward()
        if has_rev:
            rev_of(i).reverse()
    every = EVENT_EVERY if steps >= 4 * EVENT_EVERY else 1
    sampled = list(range(0, steps, every))
    ev = {i: _events(2) for i in sampled}
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        if has_rev:
            sets[i % S].forward()
            if i in ev:
                ev[i][0].record()
            rev_of(i).reverse()
            if i in ev:
                ev[i][1].record()
        else:
            if i in ev:
                ev[i][0].record()
            sets[i % S].forward()
            if i in ev:
                ev[i][1].record()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    return dt, [ev[i][0].elapsed_time(ev[i][1]) for i in sampled]


def time_each(sets, iters):
    """Per-launcher medians outside the headline region: (forward ms list, reverse ms list)."""
    import torch
    S = len(sets)
    has_rev = sets[0].has_reverse
    fwd, rev = [], []
    for i in range(iters):
        a, b = _events(2)
        a.record()
        sets[i % S].forward()
        b.record()
        fwd.append((a, b))
        if has_rev:
            c, d = _events(2)
            c.record()
            sets[(i + S // 2) % S].reverse()
            d.record()
            rev.append((c, d))
    torch.cuda.synchronize()
    return [a.elapsed_time(b) for a, b in fwd], [a.elapsed_time(b) for a, b in rev]


def graph_forward_ms(sets, replays=50):
    """Per-launch time of the forward launcher when the launches of all buffer sets are captured
    once into a HIP graph and replayed: what a launch-bound workload (cfg1: a 3 us kernel behind
    ~10 us of host-side launch work) costs once the host is out of the loop. The last replay is
    checked against the eager result."""
    import torch
    for s in sets:
        s.forward()
    torch.cuda.synchronize()
    eager = [s.y.clone() for s in sets]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for s in sets:
            s.forward()
    for s in sets:
        s.y.zero_()
    a, b = _events(2)
    graph.replay()
    torch.cuda.synchronize()
    a.record()
    for _ in range(replays):
        graph.replay()
    b.record()
    torch.cuda.synchronize()
    same = all(torch.equal(s.y, e) for s, e in zip(sets, eager))
    return a.elapsed_time(b) / (replays * len(sets)), same


def rates(w, fwd_ms, rev_ms):
    out = {"fwd_ms": round(_median(fwd_ms), 5),
           "fwd_GBps": round(w.fwd_bytes / (_median(fwd_ms) * 1e-3) / 1e9, 1)}
    out["fwd_frac"] = round(out["fwd_GBps"] / HBM_PEAK_GBPS, 4)
    out["fwd_rows_per_s"] = round(w.rows / (_median(fwd_ms) * 1e-3), 1)
    if rev_ms:
        out["rev_ms"] = round(_median(rev_ms), 5)
        out["rev_GBps"] = round(w.rev_bytes / (_median(rev_ms) * 1e-3) / 1e9, 1)
        out["rev_frac"] = round(out["rev_GBps"] / HBM_PEAK_GBPS, 4)
        out["rev_rows_per_s"] = round(w.rows / (_median(rev_ms) * 1e-3), 1)
    if hasattr(w, "fwd_flops"):
        out["fwd_TFLOPs"] = round(w.fwd_flops / (_median(fwd_ms) * 1e-3) / 1e12, 1)
        if rev_ms:
            out["rev_TFLOPs"] = round(w.rev_flops / (_median(rev_ms) * 1e-3) / 1e12, 1)
    return out


def cpu_baseline_cfg2(w, budget_s=12.0):
    """The fp64 oracle on the host cores over the same bytes: whole cfg2 passes (forward, then
    the row-parallel reverse) until about `budget_s` seconds are spent. Also returns the
    parity of the GPU results of this buffer set against that oracle."""
    import numpy as np
    import oracle_lib as O
    import gpu_lib as G
    import torch

    cores = min(O.threads(), 16)
    O.set_threads(cores)
    x, g, dy = w.x.cpu().numpy(), w.gain.cpu().numpy(), w.dy.cpu().numpy()
    passes, spent = 0, 0.0
    while True:
        t0 = time.perf_counter()
        y = O.rmsnorm_ij_j(x, g, w.eps)
        dx, dg = O.rmsnorm_ij_j_reverse_mt(x, g, dy, w.eps)
        spent += time.perf_counter() - t0
        passes += 1
        if spent >= budget_s or passes >= 4000:
            break
    gbps = passes * (w.fwd_bytes + w.rev_bytes) / spent / 1e9
    w.forward()
    w.reverse()
    torch.cuda.synchronize()
    sdx, sdg = G.rmsnorm_reverse_scales(x, g, dy, w.eps)
    G.compare(w.y, y, torch.float32, "bench cfg2 y")
    G.compare(w.dx, dx, torch.float32, "bench cfg2 dx", scale=sdx)
    G.compare(w.dgain, dg, torch.float32, "bench cfg2 dgain", rowwise=False, scale=sdg)
    return {"value": round(gbps, 3), "unit": "GB/s", "cores": cores, "kind": "port",
            "rows_per_s": round(passes * w.rows / spent, 1),
            "sample": f"{passes} full passes of cfg2 (forward + reverse, all {w.rows} rows), "
                      f"{spent:.1f} s on {cores} OpenMP threads"}, "pass (r32 1e-5 relative)"


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="cfg2", choices=sorted(SETS))
    ap.add_argument("--no-extra", action="store_true", help="skip the other workloads")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline and parity check")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this path has no multi-GPU leg (rows shard without "
                 "communication; only RMSNorm's gain gradient would need a 16 KiB all-reduce). "
                 "Run with --gpus 1.")

    import torch
    from metaphor_amd import ffi, workloads as W
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    ffi.load()  # raises if the HIP libraries are not built; there is no fallback
    torch.cuda.set_device(0)

    name = args.workload
    sets = make_sets(name)
    w = sets[0]
    dt, dom_ms = time_steps(sets, args.steps, args.warmup)
    step_bytes = w.fwd_bytes + w.rev_bytes
    value = args.steps * step_bytes / dt / 1e9
    fwd_ms, rev_ms = time_each(sets, max(20, min(args.steps, 100)))

    dom_bytes, dom_name = (w.rev_bytes, "reverse") if w.has_reverse else (w.fwd_bytes, "forward")
    avg_ms = sum(dom_ms) / len(dom_ms)
    achieved = dom_bytes / (avg_ms * 1e-3) / 1e9
    traffic = traffic_from_profile(name)

    line = {
        "metric": "achieved HBM GB/s (% of peak) + rows/s, softmax/RMSNorm/elementwise fwd+rev",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(dt / args.steps * 1e3, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": {"cfg3": "f16", "gemm": "f16"}.get(name, "f32"),
        "data": "synthetic",
        "config": {"workload": f"{name}: {W.DESCRIPTION[name]}", "buffer_sets": len(sets),
                   "bytes_per_step": step_bytes},
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBPS, 4),
        "rows_per_s": round(args.steps * w.rows / dt, 1),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": traffic,
                     "kernel": f"{name} {dom_name} launcher", "bytes_per_launch": dom_bytes,
                     "avg_launch_ms": round(avg_ms, 5), "launches_timed": len(dom_ms)},
        name: rates(w, fwd_ms, rev_ms),
    }
    if name == "cfg1":
        g_ms, same = graph_forward_ms(sets)
        line[name].update({"fwd_graph_ms": round(g_ms, 5), "fwd_graph_matches_eager": same,
                           "fwd_graph_GBps": round(w.fwd_bytes / (g_ms * 1e-3) / 1e9, 1)})

    if name in MFMA_PEAK_TFLOPS:  # the matrix product is priced in flops against the matrix cores
        tf = w.rev_flops / (avg_ms * 1e-3) / 1e12
        line["roofline"].update({"bound": "mfma", "achieved": round(tf, 1), "peak": MFMA_PEAK_TFLOPS[name],
                                 "unit": "TFLOP/s", "frac": round(tf / MFMA_PEAK_TFLOPS[name], 4),
                                 "flops_per_launch": w.rev_flops})
    if not args.no_cpu and name == "cfg2":
        line["cpu_baseline"], line["parity"] = cpu_baseline_cfg2(w)
    del sets, w
    torch.cuda.empty_cache()

    if not args.no_extra:
        extra = {}
        for other in sorted(SETS):
            if other == name:
                continue
            osets = make_sets(other)
            k = max(10, min(args.steps, 40 if other in ("cfg3", "cfg4") else 100))
            time_steps(osets, 5, 2)
            f_ms, r_ms = time_each(osets, k)
            extra[other] = rates(osets[0], f_ms, r_ms)
            extra[other]["workload"] = W.DESCRIPTION[other]
            if other == "cfg1":  # launch-bound: also the rate with the host out of the loop
                g_ms, same = graph_forward_ms(osets)
                extra[other]["fwd_graph_ms"] = round(g_ms, 5)
                extra[other]["fwd_graph_GBps"] = round(osets[0].fwd_bytes / (g_ms * 1e-3) / 1e9, 1)
                extra[other]["fwd_graph_matches_eager"] = same
            del osets
            torch.cuda.empty_cache()
        line["other_workloads"] = extra

    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
