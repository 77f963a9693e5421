#!/usr/bin/env python3
"""Benchmark of the environmental-selection hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C3|C2|C1|C4|C5] [--no-cpu] [--next-rows]

One step = one `nd_environmental_selection` call on the workload (default C3: N=20000, M=3,
D=100, topk=10000, fitness i.i.d. U[0,1) from seed 0), inputs and outputs resident in HBM.
Prints ONE JSON line.  `value` is ordered pair comparisons per second through the whole step
(N^2 / step time); the dominance kernel's own rate, the per-stage times, the roofline of the
dominant kernel and a host-CPU baseline (the CPU oracle on a bounded sample) ride along.
"""

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E
VALU_CMP_PEAK_GOPS = 39321.6  # 256 CU x 64 lanes/clk x 2.4 GHz: issue peak of v_cmp_*_f32 (not packable)
VALU_FP32_PEAK_GOPS = 78643.2  # 256 CU x 128 lanes/clk x 2.4 GHz: non-packed fp32 vector ops (157.3 TFLOP/s / 2)
FP32_VECTOR_PEAK_GFLOPS = 157300.0



def profile_traffic(workload, kernel, variant=None):
    """HBM bytes per launch of `kernel` as the committed counter summary of this workload holds them
    (profiles/<workload>_selection_hbm_traffic.md: FETCH_SIZE and WRITE_SIZE runs of this script, scaled by what the
    same counters read for a 512 MiB copy); None where the summary has no row for the kernel.  variant: words after
    the kernel's name in a summary that lists the kinds of launches of one kernel apart (else the first row counts)."""
    path = os.path.join(ROOT, "profiles", f"{workload.lower()}_selection_hbm_traffic.md")
    if not os.path.exists(path):
        return None
    for line in open(path):
        cells = [c.strip() for c in line.strip().strip("|").split("|")]
        if (len(cells) == 6 and cells[0].startswith("evx::" + kernel) and cells[0][len("evx::" + kernel):][:1] in ("", "<")
                and (variant is None or variant in cells[0])):
            try:
                return {"bytes": (float(cells[4]) + float(cells[5])) * 1e6, "read_MB": float(cells[4]),
                        "written_MB": float(cells[5]), "source": os.path.relpath(path, ROOT)}
            except ValueError:
                continue
    return None


def host_cpu():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="C3", choices=["C1", "C2", "C3", "C4", "C5"])
    ap.add_argument("--no-cpu", action="store_true", help="skip the host-CPU baseline leg")
    ap.add_argument("--cpu-sample", type=int, default=0, help="rows of the workload timed on the CPU (0 = all of them)")
    ap.add_argument("--cpu-runs", type=int, default=3, help="runs of the CPU leg (the median is reported)")
    ap.add_argument("--no-off-config", action="store_true",
                    help="skip the off-config object of the default line (one HBM-bound sweep pass at 200000 x 3)")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="also run a plain 512 MiB device copy three times, so that a rocprofv3 --pmc run of this "
                         "command holds a kernel of known traffic next to the selection kernels")
    ap.add_argument("--next-rows", action="store_true",
                    help="also time the entry points around the hot path (first-front mask, two-part selection, "
                         "tournament) and add them to the JSON line under \"next_rows\"")
    return ap.parse_args()


def median(xs):
    xs = sorted(xs)
    return xs[len(xs) // 2]


def event_time_us(fn, reps, inner=4):
    """Median duration of fn() in microseconds: HIP events on the current stream around `inner`
    back-to-back calls, so that the launch latency of the first one is amortised."""
    out = []
    for _ in range(reps):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(inner):
            fn()
        b.record()
        b.synchronize()
        out.append(a.elapsed_time(b) * 1e3 / inner)
    return median(out)


def valu_issue_rates(dev):
    """Vector issue rates that the device sustains right now, in G lane-ops/s: plain v_add_f32, v_cmp_le_f32 with
    the mask written to SGPRs, and the three-objective instruction mixes of the dominance kernel's two forms
    (vector instructions only)."""
    from evox_amd import _lib, runtime

    sink = torch.zeros(1, dtype=torch.float32, device=dev)
    s = runtime.stream_handle(dev)
    blocks, iters = 2048, 2000  # 8 waves per SIMD on 256 CUs; about half a millisecond per launch
    out = {}
    for kind, name, valu_per_iter in ((0, "v_add_f32", 16), (1, "v_cmp_to_sgpr", 16), (2, "compare_form_unit_m3", 10),
                                      (3, "arithmetic_form_unit_m3", 12)):
        def launch():
            _lib.call("evox_hip_calibration_launch", kind, blocks, iters, sink.data_ptr(), s)
        launch()
        us = event_time_us(launch, 5, inner=1)
        out[name] = blocks * 4 * iters * valu_per_iter * 64 / us / 1e3
    return out


def peel_plan(n, m):
    """(peeled from LDS?, sweeping workgroups, bytes of LDS each) as the library decides for this shape."""
    import ctypes

    from evox_amd import _lib

    out = (ctypes.c_int64 * 3)()
    _lib.call("evox_hip_peel_plan", n, m, out)
    return bool(out[0]), int(out[1]), int(out[2])


def stage_profile(w, x, f, reps):
    """Where the time of a step goes: the step's stages are run as ever longer prefixes of the pipeline, back to back
    on the launch stream (same kernels as the step's), and a stage's time is the difference between two prefixes, so
    the gaps between launches are counted where the step pays them.  The whole step is the last prefix: the selection
    entry point called through the C ABI with outputs allocated beforehand."""
    from evox_amd import _lib, runtime

    n, m = f.shape
    ws = runtime.workspace(n, m, f.device)
    s = runtime.stream_handle(f.device)
    tail = (ws.data_ptr(), ws.numel(), s)
    from_lds = peel_plan(n, m)[0]

    def prep():
        _lib.call("evox_hip_stage_prepare", f.data_ptr(), n, m, f.stride(0), f.stride(1), *tail)

    def dom():
        _lib.call("evox_hip_stage_dominance", n, m, 0, *tail)

    def count():
        _lib.call("evox_hip_stage_count", n, m, *tail)

    def peel():
        _lib.call("evox_hip_stage_peel", n, m, w.topk, None, *tail)

    xr = x if x.dim() > 1 else x.unsqueeze(1)
    out_x = torch.empty(w.topk, xr.size(1), dtype=xr.dtype, device=f.device)
    out_f = torch.empty(w.topk, m, dtype=torch.float32, device=f.device)
    out_rank = torch.empty(w.topk, dtype=torch.int32, device=f.device)
    out_dist = torch.empty(w.topk, dtype=torch.float32, device=f.device)

    def whole():
        _lib.call("evox_hip_nd_environmental_selection", xr.data_ptr(), xr.size(1) * xr.element_size(),
                  xr.stride(0) * xr.element_size(), f.data_ptr(), n, m, f.stride(0), f.stride(1), w.topk, out_x.data_ptr(),
                  out_f.data_ptr(), out_rank.data_ptr(), out_dist.data_ptr(), None, *tail)

    def upto_dom():
        prep(); dom()

    def upto_count():
        prep(); dom(); count()

    def upto_peel():
        prep(); dom()
        if not from_lds:  # (the kernel that peels from LDS counts for itself)
            count()
        peel()

    times = {"peel_from_lds": from_lds}
    whole(); upto_peel()
    torch.cuda.synchronize()
    t_prep = event_time_us(prep, reps)
    t_dom = event_time_us(upto_dom, reps)
    t_peel = event_time_us(upto_peel, reps)
    t_whole = event_time_us(whole, reps)
    times["prepare_us"] = t_prep
    times["dominance_us"] = t_dom - t_prep
    if from_lds:
        times["count_us"] = None
        times["peel_us"] = t_peel - t_dom
    else:
        t_count = event_time_us(upto_count, reps)
        times["count_us"] = t_count - t_dom
        times["peel_us"] = t_peel - t_count
    times["order_and_gather_us"] = t_whole - t_peel
    times["step_us"] = t_whole
    # the dominance stage alone, back to back (it reads what stage_prepare left and can be repeated)
    prep(); dom()
    times["dominance_alone_us"] = event_time_us(dom, reps)
    try:  # where the matrix comes from the per-objective orders: the ordering alone (an error elsewhere)
        def orders():
            _lib.call("evox_hip_stage_dominance", n, m, 5, *tail)
        orders()
        times["dominance_orders_us"] = event_time_us(orders, reps)
    except _lib.EvoxHipError:
        times["dominance_orders_us"] = None
    if times["dominance_orders_us"] is not None:
        # The selection entry point may have that stage count the dominators first and build the matrix only when front 0
        # holds fewer rows than are kept (tunable prefix_count_first; the stage entry points always do both at once):
        # the stage with the counts alone, and the whole step with the choice switched off
        with runtime.options(prefix_mode=1):
            dom()
            times["dominance_counts_only_us"] = event_time_us(dom, reps)
        with runtime.options(prefix_count_first=0):
            whole()
            times["step_matrix_always_us"] = event_time_us(whole, reps)
        # (the prefixes above are made of the stage entry points: the rest of the step is what follows them in a step
        # that launches the same kernels)
        times["order_and_gather_us"] = times["step_matrix_always_us"] - t_peel
        prep(); dom()
    upto_peel()
    runtime.note_call(ws, s)
    status = runtime.last_status()
    views = runtime.workspace_views(ws, n, m)
    rank = views["rank"].clone()
    slot_of = torch.empty(n, dtype=torch.int64, device=f.device)
    slot_of[views["orig_of"].long()] = torch.arange(n, device=f.device)
    return times, status, rank, slot_of, views["nwords"]


def cpu_baseline(w, sample_rows, runs):
    """The CPU leg, on the host's cores.  Populations whose dense relation fits host memory: the torch restatement of
    the reference's eager path, all host threads.  C5 (the reference's formulation would need 40 GB for the relation
    and two temporaries of 320 GB): the plain-C checker (OpenMP over rows), which is NOT the reference's algorithm
    (the relation as a bit matrix, peeling by counts).  Only this leg touches oracle/."""
    n = w.f.size(0) if sample_rows <= 0 else min(sample_rows, w.f.size(0))
    f = w.f[:n].contiguous()
    x = (w.x if w.x is not None else w.f)[:n].contiguous()
    k = w.topk if n == w.f.size(0) else max(1, n // 2)
    what = f"all {n} rows of {w.name}" if n == w.f.size(0) else f"first {n} rows of {w.name}"
    dense_bytes = n * n * (2 * f.size(1) + 2)  # the relation, its two (N, N, M) temporaries, one peel temporary
    secs = []
    if dense_bytes <= 24 * 2**30:
        from oracle import eager_restatement as er

        torch.set_num_threads(os.cpu_count() or 1)
        cores = torch.get_num_threads()
        for _ in range(max(1, runs)):
            t0 = time.perf_counter()
            er.environmental_selection(x, f, k)
            secs.append(time.perf_counter() - t0)
        how = "torch-CPU restatement of the reference's eager path"
    else:
        from oracle import c_oracle

        cores = c_oracle.threads()
        fn = f.numpy()
        for _ in range(max(1, runs)):
            t0 = time.perf_counter()
            c_oracle.select(fn, k)
            secs.append(time.perf_counter() - t0)
        how = (f"plain-C checker on {cores} threads: NOT the reference's algorithm (the reference's dense formulation cannot "
               "allocate at this size)")
    dt = median(secs)
    return {
        "value": n * n / dt,
        "unit": "comparisons/s",
        "cores": cores,
        "cpu": host_cpu(),
        "kind": "port",
        "sample": f"{what} (topk={k}), one nd_environmental_selection call, median of {len(secs)} run(s): {dt:.2f} s; {how}",
        "seconds": dt,
        "runs": secs,
    }


def sweep_pass_bandwidth(dev, n, m):
    """Time of the peel kernel with one sweep pass minus its time with none, over the bytes that pass reads."""
    from evox_amd import _lib, runtime, workloads

    f = workloads.uniform_population(n, m, 0, 3)[0].to(dev)
    ws = runtime.workspace(n, m, dev)
    s = runtime.stream_handle(dev)
    tail = (ws.data_ptr(), ws.numel(), s)
    with runtime.options(peel_witness=0):
        _lib.call("evox_hip_stage_prepare", f.data_ptr(), n, m, f.stride(0), f.stride(1), *tail)
        _lib.call("evox_hip_stage_dominance", n, m, 0, *tail)
        _lib.call("evox_hip_stage_count", n, m, *tail)
        _lib.call("evox_hip_stage_peel", n, m, 1, None, *tail)
        runtime.note_call(ws, s)
        front0 = runtime.last_status()["last_front_size"]

        def timed(stop):
            ts = []
            for _ in range(5):
                _lib.call("evox_hip_stage_count", n, m, *tail)
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                _lib.call("evox_hip_stage_peel", n, m, stop, None, *tail)
                b.record()
                b.synchronize()
                ts.append(a.elapsed_time(b) * 1e3)
            return median(ts)

        t_none, t_one = timed(1), timed(front0 + 1)
        views = runtime.workspace_views(ws, n, m)
        slot_of = torch.empty(n, dtype=torch.int64, device=dev)
        slot_of[views["orig_of"].long()] = torch.arange(n, device=dev)
        read = int(((((slot_of >> 6) + 2) & ~1) * 8)[views["rank"] >= 1].sum())
    runtime.release_workspaces()
    gbs = read / max(t_one - t_none, 1e-9) / 1e3
    return {"pass_us": t_one - t_none, "kernel_us_with_no_pass": t_none, "bytes": read, "bound": "hbm", "achieved": gbs,
            "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS}


def next_rows(dev, reps):
    """Times of the entry points either side of the hot path, on inputs resident in HBM."""
    from evox_amd import workloads
    from evox_amd.operators.selection import (nd_environmental_selection, nd_environmental_selection_two_part,
                                              non_dominate_rank, non_dominate_rank_until, non_dominated_mask,
                                              tournament_selection_multifit)
    from evox_amd.utils import lexsort

    out = {}
    # one sweep pass of the popcount-decrement formulation over a population where a pass is HBM-bound:
    # every row outside front 0 is read once (row_words(slot) * 8 bytes each)
    out["sweep pass N=200000 M=3"] = sweep_pass_bandwidth(dev, 200000, 3)
    # first front of a long evaluation history (what the monitor asks for) against ranking all of it
    for n, m in ((20000, 3), (200000, 3), (1000000, 3)):
        f = workloads.uniform_population(n, m, 0, 7)[0].to(dev)
        non_dominated_mask(f)
        t = event_time_us(lambda: non_dominated_mask(f), reps, inner=2)
        row = {"first_front_us": t, "front_rows": int(non_dominated_mask(f).sum())}
        if n <= 200000:
            non_dominate_rank(f)
            row["full_rank_us"] = event_time_us(lambda: non_dominate_rank(f), max(3, reps // 4), inner=1)
        out[f"first_front N={n} M={m}"] = row
        del f
    # parents + offspring: two-part entry against cat + selection (C3 split in halves)
    w = workloads.c3()
    f, x = w.f.to(dev), w.x.to(dev)
    h = f.size(0) // 2
    xa, fa, xb, fb = x[:h].clone(), f[:h].clone(), x[h:].clone(), f[h:].clone()
    nd_environmental_selection_two_part(xa, fa, xb, fb, w.topk)
    out["two_part C3"] = {
        "two_part_us": event_time_us(lambda: nd_environmental_selection_two_part(xa, fa, xb, fb, w.topk), reps),
        "cat_then_select_us": event_time_us(
            lambda: nd_environmental_selection(torch.cat([xa, xb]), torch.cat([fa, fb]), w.topk), reps),
    }
    # the cut that NSGA-III / HypE make: ranks only up to the front of the (topk+1)-th row, against all ranks
    non_dominate_rank_until(f, w.topk + 1)
    out["rank_until C3"] = {
        "rank_until_us": event_time_us(lambda: non_dominate_rank_until(f, w.topk + 1), reps),
        "full_rank_us": event_time_us(lambda: non_dominate_rank(f), reps),
    }
    # a converged population: every row on one front (the unit simplex), so the whole selection is the ordering of that
    # front by crowding distance -- what a run looks like once the front is found, which uniform fitness never shows
    for n, m in ((2000, 3), (20000, 3), (20000, 2), (50000, 3)):
        g = torch.Generator("cpu").manual_seed(5)
        fc = torch.rand(n, m, generator=g)
        fc = (fc / fc.sum(dim=1, keepdim=True)).to(dev)
        xc = torch.rand(n, 16, device=dev)
        nd_environmental_selection(xc, fc, n // 2)
        out[f"converged one front N={n} M={m} topk={n // 2}"] = {
            "us": event_time_us(lambda: nd_environmental_selection(xc, fc, n // 2), reps)}
        del fc, xc
    # many populations of more rows than the one-workgroup kernel takes, in one call (the stages of the pipeline run
    # once for all of them) against one of them alone
    from evox_amd import runtime
    for b, n, m in ((16, 4096, 3), (32, 1500, 3), (64, 2000, 2), (16, 10000, 2)):
        g = torch.Generator("cpu").manual_seed(6)
        fm = torch.rand(b, n, m, generator=g).to(dev)
        xm = torch.rand(b, n, 16, generator=g).to(dev)
        nd_environmental_selection(xm, fm, n // 2)
        nd_environmental_selection(xm[0], fm[0], n // 2)
        out[f"many populations {b} x ({n}, {m}) topk={n // 2}"] = {
            "all_in_one_call_us": event_time_us(lambda: nd_environmental_selection(xm, fm, n // 2), reps),
            "one_alone_us": event_time_us(lambda: nd_environmental_selection(xm[0], fm[0], n // 2), reps)}
        del fm, xm
    # two objectives: ranked without a dominance matrix from 4097 rows on
    for n in (50000, 200000):
        f2, x2 = workloads.uniform_population(n, 2, 16, 8)
        f2, x2 = f2.to(dev), x2.to(dev)
        nd_environmental_selection(x2, f2, n // 2)
        row = {"selection_us": event_time_us(lambda: nd_environmental_selection(x2, f2, n // 2), max(3, reps // 2), inner=1)}
        with runtime.options(two_min_rows=0):
            nd_environmental_selection(x2, f2, n // 2)
            row["selection_through_the_matrix_us"] = event_time_us(lambda: nd_environmental_selection(x2, f2, n // 2), 3, inner=1)
        out[f"two objectives N={n} topk={n // 2}"] = row
        del f2, x2
    # the selection path whose kernels never wait for each other (one launch per front), and float64 fitness, at C3
    with runtime.options(peel_stepped=1):
        nd_environmental_selection(x, f, w.topk)
        out["launch per front C3"] = {"us": event_time_us(lambda: nd_environmental_selection(x, f, w.topk), max(3, reps // 2), inner=1)}
    default_dtype = torch.get_default_dtype()
    torch.set_default_dtype(torch.float64)
    try:
        f64, x64 = f.double(), x.double()
        nd_environmental_selection(x64, f64, w.topk)
        out["float64 fitness C3"] = {"us": event_time_us(lambda: nd_environmental_selection(x64, f64, w.topk), max(3, reps // 2), inner=1)}
        del f64, x64
    finally:
        torch.set_default_dtype(default_dtype)
    # lexsort as a function of its own: HypE's lexsort([-dis, rank]) over the merged population
    full_rank = non_dominate_rank(f)
    key = torch.rand(f.size(0), device=dev)
    lexsort([key, full_rank])
    out["lexsort 2 keys x 20000"] = {"us": event_time_us(lambda: lexsort([key, full_rank]), reps)}
    # mating selection on the survivors' rank and distance (10000 binary tournaments)
    _, _, rank, dist = nd_environmental_selection(x, f, w.topk)
    tournament_selection_multifit(w.topk, [-dist, rank])
    out["tournament 10000 x 2"] = {"us": event_time_us(lambda: tournament_selection_multifit(w.topk, [-dist, rank]), reps)}
    # Monte-Carlo hypervolume: contributions of HypE (cal_hv) and the metric (100000 samples against a front)
    from evox_amd.hype import cal_hv
    from evox_amd.metrics import hv
    front = f[non_dominated_mask(f)]
    ref = torch.full((f.size(1),), 1.1, device=dev)
    cal_hv(f[:2000], ref, 1000, 10000)
    out["cal_hv 2000 points x 10000 samples"] = {"us": event_time_us(lambda: cal_hv(f[:2000], ref, 1000, 10000), reps)}
    from evox_amd import ops
    for pts, what in ((front, "first front"), (f, "whole population")):
        points = torch.abs(pts - ref)
        samples = torch.rand(100000, f.size(1), device=dev) * points.max(dim=0).values
        ops.hv_covered_count(points, samples)
        out[f"hv metric {what}: {pts.size(0)} points x 100000 samples"] = {
            "count_us": event_time_us(lambda: ops.hv_covered_count(points, samples), reps),
            "with_draws_on_default_device_us": event_time_us(lambda: hv(pts, ref), max(3, reps // 4))}
    return out


def batched_line(args, dev):
    """C4: 1024 populations of 512 rows in one call of the one-workgroup-per-population kernel.  There are no
    stages to time apart: the line carries the whole kernel, against the vector unit's issue rate."""
    from evox_amd import workloads
    from evox_amd.operators.selection import nd_environmental_selection

    w = workloads.c4()
    f = w.f.to(dev)
    batch, n, m = f.shape
    x = torch.rand(batch, n, 30, generator=torch.Generator("cpu").manual_seed(w.seed)).to(dev)

    def step():
        return nd_environmental_selection(x, f, w.topk)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / args.steps * 1e3
    # kernel time by HIP events around back-to-back launches through the C ABI on the launch stream (a ctypes call
    # costs a few microseconds, so the launches queue up and the interval per launch is the kernel's duration)
    from evox_amd import _lib, runtime

    ox, of, orank, odist = step()
    stream = runtime.stream_handle(dev)

    def launch():
        _lib.call("evox_hip_batched_nd_environmental_selection", x.data_ptr(), x.size(2) * 4, x.stride(1) * 4, x.stride(0) * 4,
                  f.data_ptr(), batch, n, m, f.stride(0), f.stride(1), f.stride(2), w.topk, ox.data_ptr(), of.data_ptr(),
                  orank.data_ptr(), odist.data_ptr(), stream)

    kernel_us = event_time_us(launch, max(5, min(args.steps, 30)), inner=8)
    pairs = float(batch) * n * n
    # every row is tested against all rows of its population (no slot order inside a workgroup):
    # m subtractions, (m - 1) ORs three at a time, clamp, shift-in per pair
    executed = (m + m // 2 + 2) * pairs
    rates = valu_issue_rates(dev)
    roofline = {"kernel": "batched_kernel", "bound": "valu", "achieved": executed / kernel_us / 1e3,
                "peak": VALU_FP32_PEAK_GOPS, "unit": "Gop/s", "frac": executed / kernel_us / 1e3 / VALU_FP32_PEAK_GOPS,
                "traffic": None, "kernel_us": kernel_us, "measured_issue_rates_Gops": rates,
                "frac_of_measured_rate": executed / kernel_us / 1e3 / rates["arithmetic_form_unit_m3"]}
    out = {
        "metric": "dominance comparisons/sec through nd_environmental_selection (N^2 ordered pairs per population and step)",
        "value": pairs / (ms_per_step * 1e-3), "unit": "comparisons/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"C4: nd_environmental_selection of {batch} populations, N={n} M={m} D=30 topk={w.topk} "
                               f"each, one launch, seed {w.seed}"},
        "latency_ms": ms_per_step, "roofline": roofline,
    }
    if not args.no_cpu:
        from oracle import eager_restatement as er

        sample = batch  # the whole workload: a few seconds of CPU work
        torch.set_num_threads(os.cpu_count() or 1)
        t0 = time.perf_counter()
        for b in range(sample):
            er.environmental_selection(x[b].cpu(), w.f[b], w.topk)
        dt = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": sample * n * n / dt, "unit": "comparisons/s", "cores": torch.get_num_threads(),
                               "kind": "port", "seconds": dt,
                               "sample": f"first {sample} populations of C4, one nd_environmental_selection call each, "
                                         f"{dt:.2f} s; torch-CPU restatement of the reference's eager path"}
        out["speedup_vs_cpu_baseline"] = out["value"] / out["cpu_baseline"]["value"]
    print(json.dumps(out))


def main():
    args = parse()
    if args.gpus != 1:
        print(f"bench.py: this build runs the selection path on ONE GPU (asked for {args.gpus}); "
              "the path is not sharded across GPUs, so there is no multi-GPU figure to report.", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs an MI355X (torch.cuda.is_available() is False)", file=sys.stderr)
        sys.exit(2)

    from evox_amd import workloads
    from evox_amd.operators.selection import nd_environmental_selection

    dev = torch.device("cuda", 0)
    if args.workload == "C4":
        batched_line(args, dev)
        return
    w = {"C1": workloads.c1, "C2": workloads.c2, "C3": workloads.c3, "C5": workloads.c5}[args.workload]()
    f = w.f.to(dev)
    x = (w.x if w.x is not None else w.f).to(dev)
    n, m = f.shape

    if args.pmc_calibration:
        src = torch.empty(512 * 2**20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    def step():
        return nd_environmental_selection(x, f, w.topk)

    # the first call of the process: kernels not yet loaded, no workspace yet, no record of an earlier selection of
    # this shape (the library keeps, per device, what the last selections found and picks the launches of the next by it)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    step()
    torch.cuda.synchronize()
    first_call_ms = (time.perf_counter() - t0) * 1e3
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    # the same steps when the library may not look at what earlier selections found (a call whose predecessor was of
    # another kind pays this launch set)
    from evox_amd import runtime as _rt
    with _rt.options(launch_memory=0):
        step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        ms_without_launch_memory = (time.perf_counter() - t0) / args.steps * 1e3

    times, status, rank, slot_of, nwords = stage_profile(w, x, f, max(5, min(args.steps, 30)))
    from_lds = times["peel_from_lds"]

    pairs = float(n) * n
    compares = 2.0 * m * pairs  # the reference's `<=` and `<` per objective and ordered pair
    # Bytes that the algorithm must move.  Rows live in slots (sorted by key) and only words 0..slot/64
    # of a row can be non-zero, so a row read costs row_words(slot) * 8 bytes.
    #   dominance: fitness in, the words of the lower triangle out (nothing above the diagonal is stored)
    #   count:     every row read once (no such stage where the rows are peeled from LDS)
    #   peel from LDS: every row read once into LDS, slot -> index table in, rank / distance fill / listing out,
    #              and one front bitmap per level
    #   peel from memory (witness pass): a row is rescanned at least once, in the pass that ranks it; plus the
    #              front bitmap (one word per 128-byte line) read by the sweepers each pass
    row_read = (((slot_of >> 6) + 2) & ~1) * 8
    passes = status["passes"]
    ranked_in_passes = (rank >= 1) & (rank <= passes)
    if from_lds:
        peel_bytes = int(row_read.sum()) + 4 * n * 4 + (passes + 1) * nwords * 8
    else:
        peel_bytes = int(row_read[ranked_in_passes].sum()) + passes * nwords * 8
    dom_bytes = n * m * 4 + int(row_read.sum())
    import ctypes

    from evox_amd import _lib

    plan = (ctypes.c_int64 * 2)()
    _lib.call("evox_hip_dominance_plan", n, m, plan)
    tile_slots = 64 * max(int(plan[0]), 2)  # dominator slots of a tile (a wave evaluates 64 rows against whole tiles)
    slots = torch.arange(n, device=rank.device)
    evaluated_pairs = float(((((slots >> 6) << 6) + 63) // tile_slots * tile_slots + tile_slots).clamp(max=nwords * 64).sum())
    # finite populations take the arithmetic form: m subtractions (scalar operand), (m - 1) ORs three at a time,
    # clamp, shift-in; others the compare form: m + 2 mask-writing instructions.  Measured alone, two-operand
    # vector-register instructions issue at about 50 T lane-ops/s and three-operand, min/max and scalar-operand
    # ones at about 32 T; mixed as in the arithmetic form they sustain about 52 T (calibration kind 3)
    finite = bool(torch.isfinite(f).all())
    # large finite populations get the matrix from the order of the rows in every objective instead (the library's
    # rule: at least 65536 rows with 3 to 8 objectives, 81920 with 2, 49152 with 9 to 16): no pairwise test is executed at all
    from_orders = finite and bool(plan[1])
    # (up to three objectives the sign of the OR is shifted in by one v_alignbit_b32 and the word complemented at the end)
    valu_per_pair = (m + (m // 2) + (1 if m <= 3 else 2)) if finite else m + 2
    executed_valu = valu_per_pair * evaluated_pairs
    executed_peak = VALU_FP32_PEAK_GOPS if finite else VALU_CMP_PEAK_GOPS
    count_bytes = int(row_read.sum()) + n * 12
    if from_orders:  # the totals that the dominance kernel left, four words per row in, four out; no row is read
        count_bytes = n * 32
    dom_us = times["dominance_alone_us"]  # the kernel by itself, back to back; "us" is its share of the step
    phases = {
        "prepare_and_slot_sort": {"us": times["prepare_us"]},
        # achieved / frac: the VALU lane-instructions this kernel issues per ordered pair of the lower triangle (tiles
        # of 64 rows x 128 or 256 columns on or below the diagonal) over the kernel's time, against the peak of the
        # instruction kind it uses.  The reference's 2*M*N^2 compares over the same time ride along as a rate only:
        # the kernel does not execute them, so no fraction of a peak is formed from them.
        "dominance": {"us": times["dominance_us"], "kernel_alone_us": dom_us, "bound": "valu",
                      "achieved": executed_valu / dom_us / 1e3, "peak": executed_peak, "unit": "G lane-ops/s",
                      "executed_form": "arithmetic" if finite else "compare",
                      "reference_compares_rate_Gcompare_s": compares / dom_us / 1e3,
                      "hbm_GBs": dom_bytes / dom_us / 1e3},
        "peel": {"us": times["peel_us"], "bound": "hbm", "achieved": peel_bytes / max(times["peel_us"], 1e-9) / 1e3,
                 "peak": HBM_PEAK_GBS, "unit": "GB/s", "passes": passes, "bytes": peel_bytes,
                 "us_per_pass": times["peel_us"] / max(passes, 1),
                 "note": ("one kernel: rows copied to LDS and counted on the way, then one exchange between all workgroups per "
                          "front, then the order of the last front; latency-bound, not bandwidth-bound") if from_lds else
                         "latency-bound: each pass is one dependent row read plus one exchange between all blocks"},
        "order_and_gather": {"us": times["order_and_gather_us"]},
    }
    if not from_lds:
        phases["count"] = {"us": times["count_us"], "bound": "hbm", "achieved": count_bytes / times["count_us"] / 1e3,
                           "peak": HBM_PEAK_GBS, "unit": "GB/s"}
    if from_orders:
        # bound by the stores of the matrix (64-byte pieces of rows that lie kilobytes apart)
        # (the stage = the ordering of the rows in every objective, then dominance_prefix_kernel: `achieved` is that
        # kernel's, its time being the stage less the ordering)
        kernel_us = dom_us - (times.get("dominance_orders_us") or 0.0)
        phases["dominance"] = {"us": times["dominance_us"], "kernel_alone_us": dom_us, "orders_us": times.get("dominance_orders_us"),
                               "prefix_kernel_us": kernel_us, "bound": "hbm", "achieved": dom_bytes / kernel_us / 1e3,
                               "peak": HBM_PEAK_GBS, "unit": "GB/s", "executed_form": "objective orders",
                               "reference_compares_rate_Gcompare_s": compares / dom_us / 1e3}
        # The selection itself counts first where its last two calls found the rows they keep in front 0 (and the peel
        # is not the one that holds the matrix in LDS): the matrix is then never written, and the kernel's launch is
        # bound by its table look-ups in LDS -- the bytes it has to move are the orders it reads and the two words per
        # row it leaves
        front0 = int((rank == 0).sum())
        counted_first = (not from_lds and front0 >= w.topk and bool(_rt.current_option("prefix_count_first", 1))
                         and bool(_rt.current_option("launch_memory", 1)) and "dominance_counts_only_us" in times)
        phases["dominance"]["front0_rows"] = front0
        phases["dominance"]["counted_first_in_the_step"] = counted_first
        if "dominance_counts_only_us" in times:
            counts_kernel_us = times["dominance_counts_only_us"] - (times.get("dominance_orders_us") or 0.0)
            counts_bytes = n * m * 8 + n * 4 + n * 8
            phases["dominance"]["counts_only"] = {
                "stage_us": times["dominance_counts_only_us"], "prefix_kernel_us": counts_kernel_us, "bytes": counts_bytes,
                "achieved": counts_bytes / counts_kernel_us / 1e3, "unit": "GB/s",
                "note": "no matrix written: bound by the look-ups in the tables that the workgroups keep in LDS"}
            phases["dominance"]["step_us_with_the_matrix_always"] = times["step_matrix_always_us"]
        if counted_first:
            phases["dominance"]["note"] = ("`us`, kernel_alone_us, prefix_kernel_us, achieved and frac are those of the launch "
                                           "that builds the matrix (stage entry point); the timed step ran the kernel for "
                                           "the counts alone (counts_only) and skipped the matrix")
    for p in phases.values():
        if "achieved" in p:
            p["frac"] = p["achieved"] / p["peak"]
    # the same executed lane-ops against what the vector unit sustains for mask-writing compares on this
    # device at the clock of the moment (the datasheet peak assumes the boost clock)
    if not from_orders:
        rates = valu_issue_rates(dev)
        phases["dominance"]["measured_issue_rates_Gops"] = rates
        phases["dominance"]["frac_of_measured_rate"] = (
            phases["dominance"]["achieved"] / (rates["v_add_f32"] if finite else rates["v_cmp_to_sgpr"]))
    # the kernel that builds the matrix: from the per-objective orders, or pair by pair -- up to eight objectives on
    # a grid that holds only the blocks at or below the diagonal (tunable dominance_folded, tiles of two or four words)
    folded = _rt.current_option("dominance_folded", 1) and m <= 8 and int(plan[0]) in (2, 4)
    dominance_kernel_name = "dominance_prefix_kernel" if from_orders else ("dominance_folded_kernel" if folded else "dominance_kernel")
    dominant = max((k for k in ("dominance", "count", "peel") if k in phases), key=lambda k: phases[k]["us"])
    d = phases[dominant]
    roofline = {
        # populations whose matrix fits the LDS of the device are peeled from there; others up to 262144 rows by the
        # record-protocol kernel, larger ones by peel_kernel
        "kernel": {"dominance": dominance_kernel_name, "count": "count_kernel",
                   "peel": "peel_lds_kernel" if from_lds else ("peel_records_kernel" if n <= 262144 else "peel_kernel")}[dominant],
        "bound": "hbm" if d["bound"] == "hbm" else "valu",
        "achieved": d["achieved"], "peak": d["peak"], "unit": d["unit"], "frac": d["frac"], "traffic": None,
        "kernel_us": d.get("prefix_kernel_us", d.get("kernel_alone_us", d["us"])),
    }
    if dominant == "dominance" and d.get("counted_first_in_the_step"):
        c = d["counts_only"]
        roofline.update({"achieved": c["achieved"], "frac": c["achieved"] / HBM_PEAK_GBS, "kernel_us": c["prefix_kernel_us"],
                         "traffic": None,
                         "note": ("the step ran this kernel for the row totals alone (front 0 held every row kept, so the "
                                  "matrix was not built): " + c["note"] + "; matrix_launch is the same kernel when it "
                                  "also writes the matrix"),
                         "matrix_launch": {"achieved": d["achieved"], "frac": d["frac"], "kernel_us": d["prefix_kernel_us"]}})
    measured = profile_traffic(args.workload, roofline["kernel"])
    if measured is not None and "matrix_launch" in roofline:  # (the first row is that of the launches with the matrix)
        roofline["matrix_launch"]["traffic"] = measured["bytes"]
        roofline["matrix_launch"]["traffic_source"] = measured["source"]
        alone = profile_traffic(args.workload, roofline["kernel"], "row totals alone")
        if alone is not None:
            roofline["traffic"] = alone["bytes"]
            roofline["traffic_source"] = alone["source"]
    elif measured is not None:
        roofline["traffic"] = measured["bytes"]
        roofline["traffic_source"] = measured["source"]
    if _rt.small_population_kernel_fits(n, m, 1):
        # a population this small is selected by one launch of the one-workgroup kernel (that is what ms_per_step
        # times); the phases and this object describe the pipeline's kernels on the same rows, timed through the
        # stage entry points
        roofline["note"] = ("the timed step is one launch of batched_kernel; phases and roofline are the pipeline's "
                            "stages on the same population")

    out = {
        "metric": "dominance comparisons/sec through nd_environmental_selection (N^2 ordered pairs per step)",
        "value": pairs / (ms_per_step * 1e-3),
        "unit": "comparisons/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": f"{w.name}: nd_environmental_selection N={n} M={m} D={x.shape[1] if x.dim() > 1 else 1} "
                               f"topk={w.topk}, fitness U[0,1) seed {w.seed}" if w.name in ("C1", "C3") else
                               f"{w.name}: nd_environmental_selection N={n} M={m} topk={w.topk} seed {w.seed}"},
        "latency_ms": ms_per_step,
        "first_call_ms": first_call_ms,
        "ms_per_step_without_launch_memory": ms_without_launch_memory,
        "step_us_by_events": times["step_us"],
        "dominance_kernel_comparisons_per_s": pairs / (times["dominance_alone_us"] * 1e-6),
        "dominance_kernel_scalar_compares_per_s": compares / (times["dominance_alone_us"] * 1e-6),
        "fronts_peeled": status["fronts"],
        "roofline": roofline,
        "phases": phases,
    }
    if args.next_rows:
        out["next_rows"] = next_rows(dev, max(5, min(args.steps, 20)))
    elif args.workload == "C3" and not args.no_off_config:
        # Not the configuration of the line and not the default formulation: the popcount-decrement sweep pass where a
        # pass is large enough to be bound by memory bandwidth (at C3 a pass would read 25 MB, 3 us at the peak, and is
        # bound by the exchange between workgroups instead, which is why the witness pass is the default there)
        runtime_ws_release = _rt.release_workspaces
        runtime_ws_release()
        out["off_config"] = {"sweep pass N=200000 M=3": sweep_pass_bandwidth(dev, 200000, 3),
                             "note": "off-config and non-default: one pass of the sweep formulation (tunable peel_witness=0) "
                                     "over a population whose passes are HBM-bound"}
    if not args.no_cpu:
        base = cpu_baseline(w, args.cpu_sample, args.cpu_runs)
        out["cpu_baseline"] = base
        out["speedup_vs_cpu_baseline"] = out["value"] / base["value"]
    print(json.dumps(out))


if __name__ == "__main__":
    main()
