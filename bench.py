#!/usr/bin/env python3
"""Benchmark of the row-reduction / elementwise hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--regions R] [--prewarm-ms P] [--workload cfg2]
                    [--no-extra] [--no-cpu] [--no-ceilings] [--strict]

A step is one pass of the hot path over one batch of the headline workload (cfg2: RMSNorm
forward + reverse, r32, [8192, 4096]) with all inputs resident in HBM: the forward of a buffer
set and then the reverse of the same set, as a training step runs them. Successive steps rotate
over several buffer sets, so that a set comes back only after the other sets' steps have passed
through the 256 MiB memory-side cache: what a reverse finds there was put there by the forward of
its own step, never by an earlier step.

Timing: W untimed warm-up steps, then a pre-warm of the same steps for a stated wall time (a
GPU that has idled runs its first milliseconds below its sustained clocks; `prewarm_ms` and
`prewarm_steps` are in the line), then R regions of EXACTLY K steps each, every region bracketed
by synchronisations. `value` is the median region's K * bytes / time, `ms_per_step` that
region's time / K; all R per-region values are in the line (`region_values_GBps`), the first
among them. Inside each region one launch of the dominant launcher is bracketed by a pair of
events on the launch stream (`in_region_launch_ms`: it includes the cost of the pair itself,
2-3 us). The roofline object's launch duration takes the pair's cost out: right after the regions,
groups of 8 steps, of 8 forwards and of 8 reverses are each timed between one pair. The reverse
inside a step is a group of steps minus a group of forwards (`roofline`), the reverse on tensors
that nothing touched recently is the third kind of group (`roofline.on_its_own`); they differ
where the reverse re-reads a tensor that its forward left in the memory-side cache.

One JSON line is printed: whole-step throughput, the roofline of the dominant launcher, and for
every workload its forward/reverse rates, roofline objects, the CPU oracle timed on the host
cores over a bounded sample of the same inputs, and the measured parity of the GPU results
against that oracle on the sample. Every roofline object also carries the rate of a plain pass
with the same reads, writes and footprint (`copy_ceiling`, from lib/libmp_probe.so), timed in
the same run.
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
SETS = {"cfg1": 16, "cfg2": 6, "cfg3": 2, "cfg4": 2, "cfg4mid": 6, "cfg5a": 3, "cfg5b": 3, "copy": 2, "permutate": 2, "gemm": 2,
        "chain": 2, "normvocab": 3}
ON_REQUEST = {"normvocab"}  # workloads outside BASELINE's configurations: run with --workload, not beside the headline
MFMA_PEAK_TFLOPS = {"gemm": 2500.0}  # dense fp16 matrix rate of the MI355X


PROFILE_OF = {"cfg1": "cfg1_softmax", "cfg2": "cfg2_rmsnorm", "cfg3": "cfg3_softmax_r16",
              "cfg4": "cfg4_fused_chain", "cfg4mid": "cfg4mid_fused_chain_kept", "cfg5a": "cfg5a_softmax_vocab", "cfg5b": "cfg5b_softmax_vocab",
              "permutate": "permutate_transpose", "gemm": "gemm_rocblas_r16",
              "chain": "chain_runtime_fused", "normvocab": "normvocab_rmsnorm_shared_rows"}


def traffic_from_profile(name, direction=None):
    """HBM bytes per launch of a launcher, as derived from the rocprofv3 FETCH_SIZE / WRITE_SIZE
    runs summarised under profiles/ (None when no summary is committed). The summaries hold
    `roofline_traffic_bytes_per_launch = N` for the dominant launcher and, where both directions
    were measured, `forward_traffic_bytes_per_launch = N` / `reverse_traffic_bytes_per_launch = N`."""
    import re
    path = os.path.join(ROOT, "profiles", f"{PROFILE_OF.get(name, name)}_hbm_traffic.md")
    if not os.path.exists(path):
        return None
    with open(path) as f:
        text = f.read()
    m = re.search(rf"{direction}_traffic_bytes_per_launch\s*=\s*(\d+)", text) if direction else None
    forward_is_dominant = "forward_traffic_bytes_per_launch" not in text  # a workload without a reverse
    if m is None and (direction in (None, "reverse") or forward_is_dominant):
        m = re.search(r"roofline_traffic_bytes_per_launch\s*=\s*(\d+)", text)
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


BATCH = 8  # launches between a pair of events: a pair costs 2-3 us of stream time, shared by the group


def _step(sets, i):
    """One step: the forward of a buffer set and then the reverse of the same set, as a training
    step runs them (the reverse re-reads what its forward read or wrote a moment ago). Steps rotate
    over the buffer sets, so a set comes back only after the other sets' steps have passed through
    the 256 MiB memory-side cache: nothing a step finds there was left by an earlier step."""
    s = sets[i % len(sets)]
    s.forward()
    if s.has_reverse:
        s.reverse()


def time_regions(sets, steps, warmup, regions=7, prewarm_s=0.25):
    """W warm-up steps, a pre-warm of the same steps for prewarm_s of wall time, then `regions`
    regions of exactly `steps` steps, each between two synchronisations. Returns the list of
    region times in seconds, the durations in ms of the one launch of the dominant launcher
    bracketed by events inside each region, and what the pre-warm took."""
    import torch
    S = len(sets)
    has_rev = sets[0].has_reverse
    for s in sets:  # every set's forward output exists before any reverse consumes it
        s.forward()
    for i in range(warmup):
        _step(sets, i)
    torch.cuda.synchronize()
    t0, n_pre = time.perf_counter(), 0
    while time.perf_counter() - t0 < prewarm_s:
        for i in range(steps):
            _step(sets, i)
        torch.cuda.synchronize()
        n_pre += steps
    prewarm = {"prewarm_ms": round((time.perf_counter() - t0) * 1e3, 1), "prewarm_steps": n_pre}
    times, pairs = [], []
    mid = steps // 2
    for _ in range(regions):
        a, b = _events(2)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            if i != mid:
                _step(sets, i)
            elif has_rev:
                sets[i % S].forward()
                a.record()
                sets[i % S].reverse()
                b.record()
            else:
                a.record()
                sets[i % S].forward()
                b.record()
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        pairs.append((a, b))
    return times, [a.elapsed_time(b) for a, b in pairs], prewarm


def time_each(sets, iters, batch=BATCH):
    """Per-launch durations in ms: groups of `batch` back-to-back launches (rotating over the buffer
    sets) between one pair of events, one value per group. Three kinds of group take turns: forwards
    only; reverses only (the rotation over the sets goes on through all groups, so a reverse works on
    a set that launches on all the other sets have passed since: nothing of it is cached); whole steps (a forward and the reverse of the same set). Returns
    the three lists (forward, reverse on its own, step); the reverse as it runs inside a step is a
    step minus a forward."""
    import torch
    S = len(sets)
    has_rev = sets[0].has_reverse
    groups = max(3, iters // batch)
    fwd, rev, step = [], [], []
    k = 0
    for _ in range(groups):
        a, b = _events(2)
        a.record()
        for _ in range(batch):
            sets[k % S].forward()
            k += 1
        b.record()
        fwd.append((a, b))
        if has_rev:
            c, d = _events(2)
            c.record()
            for _ in range(batch):  # the rotation goes on: each set was last touched S - 1 launches ago
                sets[k % S].reverse()
                k += 1
            d.record()
            rev.append((c, d))
            e, f = _events(2)
            e.record()
            for _ in range(batch):
                _step(sets, k)
                k += 1
            f.record()
            step.append((e, f))
    torch.cuda.synchronize()
    per = lambda pairs: [a.elapsed_time(b) / batch for a, b in pairs]
    return per(fwd), per(rev), per(step)


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


def native_launch_cost(launches=4000):
    """Cost of one cfg1-sized launch to a native caller: lib/host_check --launch-cost enqueues the
    softmax launcher back to back from C++ (no interpreter, no ctypes) in a child process and
    reports the host time per call and the time per launch until the stream drains."""
    import subprocess
    from metaphor_amd import ffi
    exe = os.path.join(ffi.LIB_DIR, "host_check")
    if not os.path.exists(exe):
        return None
    res = subprocess.run([exe, "--launch-cost", str(launches)], capture_output=True, text=True, timeout=120)
    if res.returncode != 0:
        return {"error": (res.stderr or res.stdout).strip()[-200:]}
    return json.loads(res.stdout.strip().splitlines()[-1])


def rates(w, fwd_ms, rev_ms, step_ms=None):
    out = {"fwd_ms": round(_median(fwd_ms), 5),
           "fwd_GBps": round(w.fwd_bytes / (_median(fwd_ms) * 1e-3) / 1e9, 1)}
    out["fwd_frac"] = round(out["fwd_GBps"] / HBM_PEAK_GBPS, 4)
    out["fwd_rows_per_s"] = round(w.rows / (_median(fwd_ms) * 1e-3), 1)
    if rev_ms:
        out["rev_ms"] = round(_median(rev_ms), 5)
        out["rev_GBps"] = round(w.rev_bytes / (_median(rev_ms) * 1e-3) / 1e9, 1)
        out["rev_frac"] = round(out["rev_GBps"] / HBM_PEAK_GBPS, 4)
        out["rev_rows_per_s"] = round(w.rows / (_median(rev_ms) * 1e-3), 1)
    if step_ms:  # a forward and the reverse of the same tensors, back to back
        out["step_ms"] = round(_median(step_ms), 5)
        out["step_GBps"] = round((w.fwd_bytes + w.rev_bytes) / (_median(step_ms) * 1e-3) / 1e9, 1)
        # the same bytes over a forward and a reverse that have nothing to do with each other (other sets):
        # what the step would run at if the reverse found nothing of its forward in the memory-side cache
        out["apart_GBps"] = round((w.fwd_bytes + w.rev_bytes) / ((_median(fwd_ms) + _median(rev_ms)) * 1e-3) / 1e9, 1)
        out["step_vs_apart"] = round(_median(step_ms) / (_median(fwd_ms) + _median(rev_ms)), 4)
    if hasattr(w, "fwd_flops"):
        out["fwd_TFLOPs"] = round(w.fwd_flops / (_median(fwd_ms) * 1e-3) / 1e12, 1)
        if rev_ms:
            out["rev_TFLOPs"] = round(w.rev_flops / (_median(rev_ms) * 1e-3) / 1e12, 1)
    return out


def reverse_in_step(fwd_ms, step_ms):
    """Durations of the reverse launcher as it runs inside a step, behind the forward of the same
    tensors: each group of steps minus the group of forwards timed next to it."""
    return [max(s - f, 1e-6) for f, s in zip(fwd_ms, step_ms)]


def roofline_of(name, direction, nbytes, launch_ms, ceiling=None, on_its_own_ms=None):
    """The roofline object of one launcher: algorithmic bytes over the average launch duration
    (events on the launch stream), against the 8 TB/s peak; `traffic` from the committed
    FETCH_SIZE / WRITE_SIZE summary (reverse launcher of workloads that have one, else forward);
    `copy_ceiling` is a plain pass with the same reads, writes and footprint, timed the same way
    in this run. With on_its_own_ms, launch_ms are the durations of a reverse inside a step (a
    step minus a forward) and on_its_own_ms those of the same launcher on tensors that nothing
    touched recently: the first is what the timed step contains, the second is the launcher against
    HBM alone (where the two differ, the reverse found a tensor of its forward in the memory-side
    cache; the plain pass of the copy ceiling never does)."""
    # an event pair also spans whatever the host does between recording the first event and
    # enqueueing the launch; a sample several times the median is such a host stall, not a launch
    med = _median(launch_ms)
    kept = [t for t in launch_ms if t <= 3.0 * med]
    avg_ms = sum(kept) / len(kept)
    achieved = nbytes / (avg_ms * 1e-3) / 1e9
    out = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
           "frac": round(achieved / HBM_PEAK_GBPS, 4),
           "traffic": traffic_from_profile(name, direction),
           "kernel": f"{name} {direction} launcher", "bytes_per_launch": nbytes,
           "avg_launch_ms": round(avg_ms, 5), "launches_timed": len(kept) * BATCH,
           "timing": f"{len(kept)} groups of {BATCH} back-to-back launches, one event pair a group",
           "host_stalls_dropped": len(launch_ms) - len(kept),
           # nothing filtered: every group counts, the slowest one shown
           "avg_launch_ms_all": round(sum(launch_ms) / len(launch_ms), 5),
           "max_launch_ms": round(max(launch_ms), 5)}
    if ceiling:
        out["copy_ceiling"] = ceiling
        out["frac_of_copy_ceiling"] = round(achieved / ceiling["GBps"], 4)
    if on_its_own_ms:
        out["kernel"] = f"{name} {direction} launcher inside a step (behind the forward of the same tensors)"
        out["timing"] = (f"{len(kept)} groups of {BATCH} steps minus {BATCH} forwards, one event pair a group of "
                         "steps and one a group of forwards")
        own = _median(on_its_own_ms)
        alone = {"avg_launch_ms": round(sum(on_its_own_ms) / len(on_its_own_ms), 5), "median_launch_ms": round(own, 5),
                 "achieved": round(nbytes / (own * 1e-3) / 1e9, 1)}
        alone["frac"] = round(alone["achieved"] / HBM_PEAK_GBPS, 4)
        if ceiling:
            alone["frac_of_copy_ceiling"] = round(alone["achieved"] / ceiling["GBps"], 4)
        out["on_its_own"] = alone
    return out


_probe = {}


def probe_lib():
    """lib/libmp_probe.so: plain passes with a workload's stream mix (measurement only)."""
    if "lib" not in _probe:
        import ctypes
        from metaphor_amd import ffi
        path = os.path.join(ffi.LIB_DIR, "libmp_probe.so")
        if not os.path.exists(path):
            raise ffi.BoundaryMissing(f"{path} is not built; run `python -m metaphor_amd.kernelgen`")
        lib = ctypes.CDLL(path)
        pp = ctypes.POINTER(ctypes.c_void_p)
        lib.mpProbeStreams.argtypes = [pp, pp, ctypes.c_int, ctypes.c_int, ffi.len_t, ctypes.c_int, ffi.StreamContext]
        lib.mpProbeStreams.restype = ctypes.c_int
        lib.mpProbeRowPairs.argtypes = [pp, ctypes.c_void_p, ctypes.c_int, ffi.len_t, ffi.len_t, ffi.StreamContext]
        lib.mpProbeRowPairs.restype = ctypes.c_int
        _probe["lib"] = lib
    return _probe["lib"]


def copy_ceiling(mix, stream_bytes, iters=24, row_pairs=None):
    """Rate of a plain pass that reads mix[0] streams and writes mix[1] streams of stream_bytes
    each: one-shot workgroups of 64 and of 256 threads, a 16-byte pack per lane and stream, and
    (row_pairs = (rows, workgroups), 16 KiB rows) the structure of the paired RMSNorm reverse
    without its arithmetic. Buffer sets rotate so that the memory-side cache cannot serve a
    repeat; timed like the launchers (groups of back-to-back launches between one event pair), median. Best shape is reported."""
    import ctypes
    import torch
    from metaphor_amd import ffi
    lib = probe_lib()
    nr, nw = mix
    per_set = (nr + nw) * stream_bytes
    sets = max(2, min(4, int((1 << 30) // per_set) + 1))
    bufs = [[torch.empty(stream_bytes, dtype=torch.uint8, device="cuda") for _ in range(nr + nw)] for _ in range(sets)]
    for bs in bufs:
        for b in bs[:nr]:
            b.view(torch.float32).normal_()  # data like the workloads': all-zero operands stream measurably faster
    arr = ctypes.c_void_p * 5
    ctx = ffi.StreamContext.from_handle(torch.cuda.current_stream().cuda_stream)
    shapes = {}

    def run(tag, launch):
        for i in range(3):
            launch(bufs[i % sets])
        pairs, k = [], 0
        for _ in range(max(3, iters // BATCH)):  # timed like the launchers: groups of back-to-back launches
            a, b = _events(2)
            a.record()
            for _ in range(BATCH):
                launch(bufs[k % sets])
                k += 1
            b.record()
            pairs.append((a, b))
        torch.cuda.synchronize()
        ms = _median([a.elapsed_time(b) / BATCH for a, b in pairs])
        shapes[tag] = round((nr + nw) * stream_bytes / (ms * 1e-3) / 1e9, 1)

    for block in (64, 256):
        def launch(bs, block=block):
            ins = arr(*[b.data_ptr() for b in bs[:nr]])
            outs = arr(*[b.data_ptr() for b in bs[nr:]])
            rc = lib.mpProbeStreams(ins, outs, nr, nw, stream_bytes, block, ctx)
            assert rc == 0, "probe refused the stream mix"
        run(f"one-shot {block} threads", launch)
    if row_pairs and nw == 1 and nr <= 2:
        rows, wgs = row_pairs

        def launch(bs):
            ins = arr(*[b.data_ptr() for b in bs[:nr]])
            rc = lib.mpProbeRowPairs(ins, bs[nr].data_ptr(), nr, rows, wgs, ctx)
            assert rc == 0
        run(f"row pairs, {wgs} workgroups of 1024", launch)
    best = max(shapes, key=shapes.get)
    del bufs
    torch.cuda.empty_cache()
    return {"GBps": shapes[best], "shape": best, "mix": f"{nr}R+{nw}W", "stream_bytes": stream_bytes,
            "buffer_sets": sets, "all_shapes_GBps": shapes}


def ceilings_for(w):
    """Copy ceilings of a workload's forward and reverse stream mixes (None for the matrix workloads)."""
    if not hasattr(w, "fwd_mix") or hasattr(w, "fwd_flops"):
        return None, None
    fb = w.fwd_bytes // sum(w.fwd_mix)
    if fb % 16:
        return None, None
    pairs = None
    if w.name == "cfg2":
        pairs = (w.shape[0], 256)
    fwd = copy_ceiling(w.fwd_mix, fb, row_pairs=pairs)
    rev = copy_ceiling(w.rev_mix, w.rev_bytes // sum(w.rev_mix), row_pairs=pairs) if w.has_reverse else None
    return fwd, rev


def _numbers(got, ref, dtype, rowwise=True, scale=None, atol=None):
    """n, max_abs, max_rel, violations of one comparison under this path's bound (tests/gpu_lib.py)."""
    import gpu_lib as G
    st = G.parity_stats(got, ref, dtype, rowwise=rowwise, scale=scale, atol=atol)
    return {"n": st["n"], "max_abs": float(f"{st['max_abs']:.3e}"), "max_rel": float(f"{st['max_rel']:.3e}"),
            "violations": st["violations"]}


BOUND_TEXT = {
    "r32": "|got - ref| <= 1e-5 * max(|ref|, RMS(ref row or tensor)); softmax outputs: <= 1e-6 absolute",
    "r16": "|got - ref| <= 2e-3 * max(|ref|, RMS(ref row)) + 2^-24",
}


def cpu_and_parity(name, w, budget_s):
    """The fp64 oracle (oracle/mp_oracle.c, OpenMP) on the host cores over a bounded sample of the
    workload's own input bytes, repeated until about budget_s seconds are spent, and the measured
    parity of the GPU results of this buffer set against the oracle on that sample. The sample:
    cfg1 and cfg2 whole; cfg3 the first four 2048-row blocks; cfg4 / chain the first 2^22 elements;
    cfg5a the first 32 rows, cfg5b the first 96. Returns (cpu_baseline, parity); every comparison
    also raises when an entry is outside its bound."""
    import numpy as np
    import oracle_lib as O
    import gpu_lib as G
    import torch

    avail = os.cpu_count() or 1
    used = min(O.threads(), avail)  # OMP_NUM_THREADS where the box sets it (its share of the host per GPU)
    O.set_threads(used)
    w.forward()
    if w.has_reverse:
        w.reverse()
    torch.cuda.synchronize()
    dt = w.dtype
    tol = G.softmax_tol(dt)
    parity = {"reference": "fp64 oracle (oracle/mp_oracle.c) on the same input bytes",
              "bound": BOUND_TEXT["r16" if dt == torch.float16 else "r32"]}

    if name == "cfg2":
        x, g, dy = w.x.cpu().numpy(), w.gain.cpu().numpy(), w.dy.cpu().numpy()
        sample, units = f"whole problem, all {w.rows} rows, forward + reverse", w.rows
        nbytes = w.fwd_bytes + w.rev_bytes

        def once():
            return O.rmsnorm_ij_j(x, g, w.eps), O.rmsnorm_ij_j_reverse_mt(x, g, dy, w.eps)

        def check(res):
            y, (dx, dg) = res
            sdx, _ = G.rmsnorm_reverse_scales(x, g, dy, w.eps)
            G.compare(w.y, y, dt, "bench cfg2 y")
            G.compare(w.dx, dx, dt, "bench cfg2 dx", scale=sdx)
            G.compare(w.dgain, dg, dt, "bench cfg2 dgain", rowwise=False)
            parity.update({"y": _numbers(w.y, y, dt), "dx": _numbers(w.dx, dx, dt),
                           "dgain": _numbers(w.dgain, dg, dt, rowwise=False),
                           "dx_with_cancellation_scale": _numbers(w.dx, dx, dt, scale=sdx)})
    elif name in ("cfg1", "cfg3", "cfg5a", "cfg5b"):
        m, n = w.shape
        rows = {"cfg1": m, "cfg3": min(m, 4 * w.block) if name == "cfg3" else 0, "cfg5a": 32, "cfg5b": 96}[name]
        rows = min(rows, m)
        x = w.x[:rows].cpu().numpy()
        es = w.x.element_size()
        units = rows
        if w.has_reverse:
            yg, dy = w.y[:rows].cpu().numpy(), w.dy[:rows].cpu().numpy()
            sample = f"rows 0..{rows - 1} of {m}, forward + reverse (the reverse reads the GPU's own forward output)"
            nbytes = 5 * rows * n * es

            def once():
                return O.softmax_ij_j(x), O.softmax_ij_j_reverse(yg, dy)

            def check(res):
                y, dx = res
                sc = G.softmax_reverse_scale(yg, dy)
                G.compare(w.y[:rows], y, dt, f"bench {name} y", **tol)
                G.compare(w.dx[:rows], dx, dt, f"bench {name} dx", scale=sc)
                parity.update({"y": _numbers(w.y[:rows], y, dt, **tol), "dx": _numbers(w.dx[:rows], dx, dt),
                               "dx_with_cancellation_scale": _numbers(w.dx[:rows], dx, dt, scale=sc)})
        else:
            sample = f"rows 0..{rows - 1} of {m}, forward"
            nbytes = 2 * rows * n * es

            def once():
                return O.softmax_ij_j(x)

            def check(y):
                G.compare(w.y[:rows], y, dt, f"bench {name} y", **tol)
                parity.update({"y": _numbers(w.y[:rows], y, dt, **tol)})
    elif name in ("cfg4", "cfg4mid", "chain"):
        k = min(w.n, 1 << 22)
        ins = [t[:k].cpu().numpy() for t in (w.a, w.b, w.c, w.d)]
        de = w.de[:k].cpu().numpy()
        sample, units, nbytes = f"elements 0..{k - 1} of {w.n}, forward + reverse", k, 56 * k
        if name in ("cfg4", "cfg4mid"):
            def once():
                return O.fused_selu_hadamard_add_add(*ins), O.fused_selu_hadamard_add_add_reverse(*ins, de)
        else:  # relu((a - b) * (c + d)) and its gradients in fp64 (relu's convention: zero counts as positive)
            def once():
                a64, b64, c64, d64 = (t.astype(np.float64) for t in ins)
                u, v = a64 - b64, c64 + d64
                p = u * v
                g = de.astype(np.float64) * (p >= 0)
                return np.where(p >= 0, p, 0.0), (g * v, -(g * v), g * u, g * u)

        def check(res):
            e, grads = res
            G.compare(w.e[:k], e, dt, f"bench {name} e", rowwise=False)
            parity["e"] = _numbers(w.e[:k], e, dt, rowwise=False)
            for tag, got, ref in zip("abcd", (w.da, w.db, w.dc, w.dd), grads):
                G.compare(got[:k], ref, dt, f"bench {name} d{tag}", rowwise=False)
                parity["d" + tag] = _numbers(got[:k], ref, dt, rowwise=False)
    else:
        return None, None

    passes, spent, res = 0, 0.0, None
    while True:
        t0 = time.perf_counter()
        res = once()
        spent += time.perf_counter() - t0
        passes += 1
        if spent >= budget_s or passes >= 100000:
            break
    check(res)
    if name == "chain":  # numpy stands in for the oracle here: a parity check, not a baseline
        parity["reference"] = "numpy fp64 on the same input bytes"
        return None, parity
    cpu = {"value": round(passes * nbytes / spent / 1e9, 3), "unit": "GB/s", "cores": used, "kind": "port",
           "threads_used": used, "cores_available": avail,
           "rows_per_s": round(passes * units / spent, 1),
           "sample": f"{passes} passes over {sample}; {spent:.1f} s on {used} OpenMP threads "
                     f"({avail} logical cores visible; the thread count is the box's OMP_NUM_THREADS, its share of the host per GPU)"}
    return cpu, parity


CPU_BUDGET_S = {"cfg2": 10.0, "cfg1": 1.5, "cfg3": 3.0, "cfg4": 3.0, "cfg4mid": 1.0, "chain": 1.5, "cfg5a": 3.0, "cfg5b": 3.0}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--regions", type=int, default=7, help="timed regions of --steps steps each; value = the median one")
    ap.add_argument("--prewarm-ms", type=float, default=250.0,
                    help="wall time of the disclosed pre-warm in front of the regions (counter runs under rocprofv3 use 0)")
    ap.add_argument("--workload", default="cfg2", choices=sorted(SETS))
    ap.add_argument("--sets", type=int, default=0, help="buffer sets the steps rotate over (default: the workload's own number)")
    ap.add_argument("--no-extra", action="store_true", help="skip the other workloads")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline and parity check")
    ap.add_argument("--no-ceilings", action="store_true", help="skip the plain-copy ceilings of each stream mix")
    ap.add_argument("--strict", action="store_true", help="exit 1 when a recorded check fails (a run-time chain slower than the build-time one)")
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

    import contextlib
    name = args.workload
    sets = make_sets(name, args.sets or None)
    w = sets[0]
    times, in_region_ms, prewarm = time_regions(sets, args.steps, args.warmup, args.regions, args.prewarm_ms * 1e-3)
    step_bytes = w.fwd_bytes + w.rev_bytes
    region_values = [args.steps * step_bytes / t / 1e9 for t in times]
    dt = _median(times)  # the median region: `value` and `ms_per_step` describe the same region
    value = args.steps * step_bytes / dt / 1e9
    fwd_ms, rev_ms, step_ms = time_each(sets, max(24, min(args.steps, 96)))

    dom_bytes, dom_name, dom_ms = (w.rev_bytes, "reverse", reverse_in_step(fwd_ms, step_ms)) if w.has_reverse else (w.fwd_bytes, "forward", fwd_ms)
    checks_failed = []
    cpu_line = parity = None
    if not args.no_cpu:
        with contextlib.redirect_stdout(sys.stderr):  # stdout carries the one JSON line only
            cpu_line, parity = cpu_and_parity(name, w, CPU_BUDGET_S.get(name, 3.0))
    per_workload = rates(w, fwd_ms, rev_ms, step_ms)
    del sets
    torch.cuda.empty_cache()
    fwd_ceiling, rev_ceiling = (None, None) if args.no_ceilings else ceilings_for(w)

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
        "config": {"workload": f"{name}: {W.DESCRIPTION[name]}", "buffer_sets": args.sets or SETS[name],
                   "bytes_per_step": step_bytes},
        # how `value` was taken: median of `regions` regions of `steps` steps each, after the warm-up
        # steps and a disclosed pre-warm of the same steps; the first region is region_values_GBps[0]
        "regions": args.regions,
        "region_values_GBps": [round(v, 1) for v in region_values],
        **prewarm,
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBPS, 4),
        "rows_per_s": round(args.steps * w.rows / dt, 1),
        # the dominant launcher: groups of back-to-back launches between event pairs, right after the regions
        "roofline": roofline_of(name, dom_name, dom_bytes, dom_ms, rev_ceiling if w.has_reverse else fwd_ceiling,
                                on_its_own_ms=rev_ms if w.has_reverse else None),
        name: per_workload,
    }
    # one launch of the dominant launcher inside each timed region, events around it (pair included)
    line["roofline"]["in_region_launch_ms"] = [round(t, 5) for t in in_region_ms]
    if w.has_reverse:
        line[name]["roofline_fwd"] = roofline_of(name, "forward", w.fwd_bytes, fwd_ms, fwd_ceiling)
    avg_ms = line["roofline"]["avg_launch_ms"]
    if name == "cfg1":
        g_sets = make_sets(name)
        g_ms, same = graph_forward_ms(g_sets)
        line[name].update({"fwd_graph_ms": round(g_ms, 5), "fwd_graph_matches_eager": same,
                           "fwd_graph_GBps": round(w.fwd_bytes / (g_ms * 1e-3) / 1e9, 1),
                           "native_caller": native_launch_cost()})
        del g_sets

    if name in MFMA_PEAK_TFLOPS:  # the matrix product is priced in flops against the matrix cores
        tf = w.rev_flops / (avg_ms * 1e-3) / 1e12
        line["roofline"].update({"bound": "mfma", "achieved": round(tf, 1), "peak": MFMA_PEAK_TFLOPS[name],
                                 "unit": "TFLOP/s", "frac": round(tf / MFMA_PEAK_TFLOPS[name], 4),
                                 "flops_per_launch": w.rev_flops})
    if cpu_line is not None:
        line["cpu_baseline"] = cpu_line
    if parity is not None:
        line["parity"] = parity
    del w
    torch.cuda.empty_cache()

    if not args.no_extra:
        extra = {}
        for other in sorted(SETS):
            if other == name or other in ON_REQUEST:
                continue
            osets = make_sets(other)
            o = osets[0]
            # launches timed per direction (groups of 8): independent of --steps, which sizes the headline's regions
            k = 40 if other in ("cfg3", "cfg4", "chain", "gemm", "permutate", "copy") else 96
            t_warm = time.perf_counter()  # the same pre-warm as the headline gets, shorter
            while time.perf_counter() - t_warm < 0.05:
                for i in range(4):
                    _step(osets, i)
                torch.cuda.synchronize()
            f_ms, r_ms, s_ms = time_each(osets, k)
            extra[other] = rates(o, f_ms, r_ms, s_ms)
            extra[other]["workload"] = W.DESCRIPTION[other]
            if other == "cfg1":  # launch-bound: also the rate with the host out of the loop
                g_ms, same = graph_forward_ms(osets)
                extra[other]["fwd_graph_ms"] = round(g_ms, 5)
                extra[other]["fwd_graph_GBps"] = round(o.fwd_bytes / (g_ms * 1e-3) / 1e9, 1)
                extra[other]["fwd_graph_matches_eager"] = same
                extra[other]["native_caller"] = native_launch_cost()
            if not args.no_cpu and other in CPU_BUDGET_S:
                with contextlib.redirect_stdout(sys.stderr):
                    o_cpu, o_parity = cpu_and_parity(other, o, CPU_BUDGET_S[other])
                if o_cpu is not None:
                    extra[other]["cpu_baseline"] = o_cpu
                if o_parity is not None:
                    extra[other]["parity"] = o_parity
            del osets
            torch.cuda.empty_cache()
            if other.startswith("cfg") or other == "chain":  # the same roofline object as the headline workload carries
                f_ceil, r_ceil = (None, None) if args.no_ceilings or other == "cfg1" else ceilings_for(o)
                if o.has_reverse:
                    extra[other]["roofline"] = roofline_of(other, "reverse", o.rev_bytes, reverse_in_step(f_ms, s_ms), r_ceil,
                                                           on_its_own_ms=r_ms)
                    extra[other]["roofline_fwd"] = roofline_of(other, "forward", o.fwd_bytes, f_ms, f_ceil)
                else:
                    extra[other]["roofline"] = roofline_of(other, "forward", o.fwd_bytes, f_ms, f_ceil)
            del o
            torch.cuda.empty_cache()
        # an expression compiled at run time must run at the rate of the build-time chain with the
        # same streams (same engine, same launch plan): within 10 % in both directions
        if "chain" in extra and "cfg4" in extra:
            c, f = extra["chain"], extra["cfg4"]
            ratio = {"fwd": round(c["fwd_ms"] / f["fwd_ms"], 4), "rev": round(c["rev_ms"] / f["rev_ms"], 4)}
            ok = all(v <= 1.10 for v in ratio.values())
            extra["chain"]["runtime_vs_buildtime_ms_ratio"] = {**ratio, "bound": 1.10, "ok": ok}
            if not ok:
                checks_failed.append(f"run-time chain slower than the build-time chain: {ratio}")
        line["other_workloads"] = extra
    line["checks_failed"] = checks_failed

    print(json.dumps(line), flush=True)
    for msg in checks_failed:
        print(f"bench.py: CHECK FAILED: {msg}", file=sys.stderr)
    if checks_failed and args.strict:
        sys.exit(1)


if __name__ == "__main__":
    main()
