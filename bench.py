#!/usr/bin/env python3
"""Benchmark of the custom-op hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One timed "step" is the headline workload (cfg2): BinnedSelectKnn on one
HGCal-like event of N=150,000 hits with 4-D coordinates and K=64 (bounding box,
binning, grouping by bin, search, un-sort — everything the wrapper does),
followed by the AccumulateKnn forward over F=64 features with ten times the
returned squared distances (weights exp(-10 d^2), what the reference's GravNet
passes). Inputs are resident in HBM before the timed region. `value`
is kNN queries per second of the whole step. The step is timed twice over K
iterations each: launched op by op, and as a replay of the step captured once
into a HIP graph (same kernels, same buffers); the faster of the two is reported
(the replay only when its outputs equal the eager ones), `config.launch` says which, and
`config.eager_ms_per_step` keeps the other number.

The `roofline` object is measured in a second timed loop of the same run (also
K iterations, HIP events on the stream the kernels are launched on) at cfg4
(N=1,000,000, K=64, F=128, banded neighbour table): the dominant piece, one call
of the accumulate_knn gradient (algorithmic bytes 4*N*(3K+5F); two kernels: the
streaming pass that builds the per-slot hit records and the gather over the
inverse index), with the forward launch (4*N*(2K+4F)), the forward+gradient pair
and the pair plus one build of the inverse neighbour index next to it, against
the 8 TB/s HBM peak. Next to the fraction of the HBM roofline it states two
floors of what this formulation can reach on this memory system: the same
K-fold gather of 512-byte rows with one multiply-add per element and nothing
else (`l2_gather_floor_ms`: PushKnn over the same table, timed in the same run),
and the issue time of the gradient's vector instructions alone (`valu_floor_ms`,
from the committed counter summary).

`cpu_baseline` times the CPU oracle (a single-threaded C restatement of the
reference CPU kernels) on this box's host: the binned kNN kernel over the full
cfg2 event.

Prints ONE JSON line on stdout; progress goes to stderr.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(1, os.path.join(ROOT, "tests"))  # workloads.py: the seeded inputs shared with the tests

HBM_PEAK_GBS = 8000.0

# HBM bytes per launch at full cfg4 come from two hardware-counter runs of this file's
# roofline section (FETCH_SIZE, WRITE_SIZE, scaled by what the counters read for the 512 MB
# calibration copy below). Counters cannot be read from inside the timed run, so the line
# carries what the committed summary profiles/accumulate_knn_cfg4_hbm_counters.txt holds
# (its "bench.py reads" line, stamped with the commit it was measured at), or null.
TRAFFIC_SUMMARY = os.path.join(ROOT, "profiles", "accumulate_knn_cfg4_hbm_counters.txt")
COUNTER_SUMMARY = os.path.join(ROOT, "profiles", "accumulate_knn_cfg4_sq_tcc_counters.txt")


def measured_valu_floor():
    """{'ms': issue time of the gradient's vector instructions, 'measured_at': commit} from the committed
    counter summary (its "bench.py reads" line), or None"""
    try:
        with open(COUNTER_SUMMARY) as f:
            for line in f:
                if line.startswith("bench.py reads:"):
                    fields = dict(kv.split("=", 1) for kv in line.split(":", 1)[1].split())
                    return {"ms": float(fields["gradient_valu_floor_ms"]), "measured_at": fields.get("measured_at", "unknown")}
    except (OSError, KeyError, ValueError):
        pass
    return None


def measured_traffic():
    """{'forward': bytes, 'gradient': bytes, 'measured_at': commit} from the committed summary, or None"""
    try:
        with open(TRAFFIC_SUMMARY) as f:
            for line in f:
                if line.startswith("bench.py reads:"):
                    fields = dict(kv.split("=", 1) for kv in line.split(":", 1)[1].split())
                    return {"forward": float(fields["forward_bytes"]), "gradient": float(fields["gradient_bytes"]),
                            "measured_at": fields.get("measured_at", "unknown")}
    except (OSError, KeyError, ValueError):
        pass
    return None


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def event_ms(fn, steps, warmup):
    """average milliseconds per call with HIP events on torch's current stream"""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    times = []
    for _ in range(steps):
        a = torch.cuda.Event(enable_timing=True)
        b = torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        b.synchronize()
        times.append(a.elapsed_time(b))
    return float(np.mean(times)), float(np.median(times)), float(np.min(times))


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline_knn(cfg, reps=5, opt_level_0=False):
    """the oracle's binned kNN kernel over all queries of cfg2, `reps` passes, one thread
    (opt_level_0: built without optimisation, the flags of the reference's own Makefile)"""
    import oracle
    coords, rs, K = cfg["coords"], cfg["row_splits"], cfg["K"]
    dbin, flat, nb, bw, nper = oracle.BinByCoordinates(coords[:, :3], rs, n_bins=cfg["n_bins"])
    order = np.argsort(flat, kind="stable")
    bb = np.concatenate([[0], np.cumsum(nper)]).astype(np.int32)
    sc, sf, sd = coords[order], flat[order], dbin[order]
    t0 = time.perf_counter()
    for _ in range(reps):
        oracle.binned_select_knn_kernel(K, sc, sf, sd, bb, nb, bw, opt_level_0=opt_level_0)
    dt = time.perf_counter() - t0
    return reps * len(coords) / dt, dt


def cpu_baseline_accumulate(cfg4_small):
    import oracle
    w = np.exp(-cfg4_small["distsq"]).astype(np.float32)
    t0 = time.perf_counter()
    _, arg = oracle.accumulate_knn_kernel(w, cfg4_small["features"], cfg4_small["indices"])
    t1 = time.perf_counter()
    oracle.accumulate_knn_grad_kernel(cfg4_small["grad_out"], w, cfg4_small["features"], cfg4_small["indices"], arg)
    t2 = time.perf_counter()
    return t1 - t0, t2 - t1


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # the headline step takes 0.6 ms: a few hundred untimed steps bring clocks and caches to their steady state (a
    # cold process reads about 6 % slower over its first few dozen steps)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=300)
    ap.add_argument("--skip-cpu-baseline", action="store_true")
    ap.add_argument("--roofline-scale", type=float, default=1.0, help="shrink cfg4 (debugging only)")
    ap.add_argument("--section", choices=["all", "headline", "roofline", "streams", "condensates", "blob"], default="all",
                    help="run only one part (for profiling); the JSON line is printed for 'all' only. 'streams': the "
                         "cfg4 gradient next to its variants without the max half and without the weight gradient, "
                         "whose counter differences split its L2 requests by data stream. 'condensates': cfg5 alone, both "
                         "assignment modes. 'blob': the kNN search over the 4-D Gaussian blob alone")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build targets ONE GPU (no collectives, no sharding); run with --gpus 1. "
                 "Events are independent, so several GPUs would each take whole events.")

    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    from hgcalml_amd import AccumulateKnn, AccumulateLinKnn, BinnedSelectKnn, BuildAndAssignCondensatesBinned, ops
    import workloads
    dev = "cuda:0"
    torch.cuda.set_device(0)

    if args.section == "condensates":
        c5 = workloads.cfg5(ragged=True)
        a5 = [torch.from_numpy(c5[k]).to(dev) for k in ("ccoords", "betas", "dist", "row_splits")]
        for mode in (True, False):
            m5 = event_ms(lambda: BuildAndAssignCondensatesBinned(*a5, c5["beta_threshold"], assign_by_max_beta=mode),
                          args.steps, args.warmup)
            log("bench: cfg5 condensates (%s) %.3f ms" % ("max-beta" if mode else "min-distance", m5[0]))
        return
    if args.section == "blob":
        blob = torch.from_numpy(np.random.default_rng(5).standard_normal((150000, 4)).astype(np.float32)).to(dev)
        rs_blob = torch.tensor([0, 150000], dtype=torch.int32, device=dev)
        mb = event_ms(lambda: BinnedSelectKnn(65, blob, rs_blob, n_bins=30), args.steps, args.warmup)
        log("bench: kNN over a 4-D Gaussian blob, N=150000, K=65: %.3f ms" % mb[0])
        return
    # ------------------------------------------------------------------ headline: cfg2
    c2 = workloads.cfg2()
    n2, K2 = len(c2["coords"]), c2["K"]
    if args.section not in ("roofline", "streams"):
        coords = torch.from_numpy(c2["coords"]).to(dev)
        rs = torch.from_numpy(c2["row_splits"]).to(dev)
        feat = torch.from_numpy(c2["features"]).to(dev)
        state = {}

        def step():
            idx, dist = BinnedSelectKnn(K2, coords, rs, n_bins=c2["n_bins"])
            out, _ = AccumulateKnn(10. * dist, feat, idx)  # the callers' weights exp(-10 d^2) (GravNetLayersRagged.py:3269)
            state["idx"], state["dist"], state["out"] = idx, dist, out

        log("bench: warmup + %d timed steps of cfg2 (kNN N=%d 4-D K=%d + accumulate fwd F=64)" % (args.steps, n2, K2))
        for _ in range(args.warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        eager_ms_per_step = wall / args.steps * 1e3
        ms_per_step, launch_mode = eager_ms_per_step, "eager (one launch sequence per step)"

        # The same step captured once into a HIP graph and replayed: identical kernels on
        # identical buffers, without the per-step launch sequence. Taken as the headline
        # only if the replayed outputs equal the eager ones bit for bit.
        try:
            eager = {k: v.clone() for k, v in state.items()}
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side), torch.no_grad():
                step()
            torch.cuda.current_stream().wait_stream(side)
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph), torch.no_grad():
                step()
            captured = dict(state)
            for _ in range(args.warmup):
                graph.replay()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(args.steps):
                graph.replay()
            torch.cuda.synchronize()
            graph_ms_per_step = (time.perf_counter() - t0) / args.steps * 1e3
            if all(torch.equal(captured[k], eager[k]) for k in eager):
                if graph_ms_per_step < eager_ms_per_step:
                    ms_per_step, launch_mode = graph_ms_per_step, "HIP graph replay of the captured step"
                else:
                    launch_mode = "eager (a HIP graph replay of the step took %.4f ms)" % graph_ms_per_step
            else:
                log("bench: graph replay differs from the eager step; keeping the eager time")
            step()  # eager again: later sections read state[...]
            torch.cuda.synchronize()
        except Exception as e:  # capture unsupported: the eager number stands
            log("bench: HIP graph capture failed (%r); keeping the eager time" % (e,))
        value = n2 / (ms_per_step * 1e-3)

        knn_ms = event_ms(lambda: BinnedSelectKnn(K2, coords, rs, n_bins=c2["n_bins"]), args.steps, 2)
        idx2, dist2 = state["idx"], state["dist"]
        acc2_ms = event_ms(lambda: AccumulateKnn(10. * dist2, feat, idx2), args.steps, 2)
        log("bench: cfg2 step %.3f ms [%s; eager %.3f ms] (kNN op %.3f ms, accumulate fwd %.3f ms)" %
            (ms_per_step, launch_mode, eager_ms_per_step, knn_ms[0], acc2_ms[0]))

    if args.section == "headline":
        return
    # ------------------------------------------------------------------ roofline: cfg4 accumulate fwd + grad
    log("bench: generating cfg4 (N=1M, K=64, F=128) ...")
    c4 = workloads.cfg4(scale=args.roofline_scale)
    n4, K4, F4 = len(c4["indices"]), c4["K"], c4["F"]
    w4 = torch.exp(-torch.from_numpy(c4["distsq"]).to(dev))
    x4 = torch.from_numpy(c4["features"]).to(dev)
    i4 = torch.from_numpy(c4["indices"]).to(dev)
    g4 = torch.from_numpy(c4["grad_out"]).to(dev)
    # known-size device copy (512 MB read + 512 MB write): calibrates FETCH_SIZE / WRITE_SIZE
    # when this run is profiled with hardware counters
    copy_dst = torch.empty_like(x4)
    copy_ms = event_ms(lambda: copy_dst.copy_(x4), 3, 1)
    log("bench: calibration copy of %.0f MB: %.3f ms (%.0f GB/s read+write)" %
        (x4.numel() * 4 / 1e6, copy_ms[0], 2 * x4.numel() * 4 / (copy_ms[0] * 1e-3) / 1e9))
    del copy_dst
    # launches of milliseconds: a handful of calls is a steady measurement
    r_steps, r_warm = min(args.steps, 20), min(args.warmup, 5)
    fwd_ms = event_ms(lambda: torch.ops.hgcalml.accumulate_knn_slots(w4, x4, i4, 0, True), r_steps, r_warm)
    _, arg4, slots4 = torch.ops.hgcalml.accumulate_knn_slots(w4, x4, i4, 0, True)
    inv_ms = event_ms(lambda: ops.inverse_neighbour_index(i4), 3, 1)
    inv = ops.inverse_neighbour_index(i4)
    import hgcalml_amd.globals as gl
    grad_ms = event_ms(lambda: torch.ops.hgcalml.accumulate_knn_grad_slots(g4, w4, x4, i4, arg4, slots4, *inv),
                       r_steps, r_warm)
    # the same gradient through the gather that compares slot bytes (no records, no streaming pass)
    gl.acc_grad_hit_records = False
    grad_slots_ms = event_ms(lambda: torch.ops.hgcalml.accumulate_knn_grad_slots(g4, w4, x4, i4, arg4, slots4, *inv),
                             max(3, r_steps // 2), 2)
    gl.acc_grad_hit_records = None
    # the K-fold gather of this table with one multiply-add per gathered element and nothing else
    push_ms = event_ms(lambda: torch.ops.hgcalml.push_knn(w4, x4, i4), max(3, r_steps // 2), 2)
    bytes_fwd = 4.0 * n4 * (2 * K4 + 4 * F4)
    bytes_bwd = 4.0 * n4 * (3 * K4 + 5 * F4)
    achieved = (bytes_fwd + bytes_bwd) / ((fwd_ms[0] + grad_ms[0]) * 1e-3) / 1e9
    log("bench: cfg4 fwd %.3f ms, grad %.3f ms (slot-byte gather %.3f ms, bare ordered gather %.3f ms), inverse index "
        "(one-off) %.3f ms -> %.1f GB/s" % (fwd_ms[0], grad_ms[0], grad_slots_ms[0], push_ms[0], inv_ms[0], achieved))

    if args.section == "streams":
        # same table, same inputs: the gradient without the max half (no slot bytes, no max-half loads), and the
        # ordered gather alone (push_knn: mean-half rows, weights and inverse slots; no own feature row, no
        # weight-gradient writes)
        g4_mean = g4[:, :F4].contiguous()
        for _ in range(max(2, r_steps)):
            torch.ops.hgcalml.accumulate_knn_grad_slots(g4_mean, w4, x4, i4, arg4, slots4, *inv)
            torch.ops.hgcalml.push_knn(w4, g4_mean, i4)
        torch.cuda.synchronize()
        return
    if args.section == "roofline":
        return
    # ------------------------------------------------------------------ information: cfg3, cfg5
    extra = {}
    try:
        c3 = workloads.cfg3()
        co3, rs3 = torch.from_numpy(c3["coords"]).to(dev), torch.from_numpy(c3["row_splits"]).to(dev)
        # sub-millisecond, instruction-bound calls: warmed up like the headline loop (see --warmup)
        m3 = event_ms(lambda: BinnedSelectKnn(c3["K"], co3, rs3, n_bins=c3["n_bins"], max_radius=c3["max_radius"]), 30, 100)
        extra["cfg3_knn_ms"] = round(m3[0], 3)
        extra["cfg3_queries_per_s"] = round(len(c3["coords"]) / (m3[0] * 1e-3), 1)
        # a 4-D Gaussian blob (the shape of a learned coordinate space): N=150k, K=65
        blob = torch.from_numpy(np.random.default_rng(5).standard_normal((150000, 4)).astype(np.float32)).to(dev)
        mb = event_ms(lambda: BinnedSelectKnn(65, blob, rs, n_bins=30), 30, 150)
        extra["knn_gaussian_blob_4d_N150k_K65_ms"] = round(mb[0], 3)
        c5 = workloads.cfg5(ragged=True)
        a5 = [torch.from_numpy(c5[k]).to(dev) for k in ("ccoords", "betas", "dist", "row_splits")]
        for mode in (True, False):
            m5 = event_ms(lambda: BuildAndAssignCondensatesBinned(*a5, c5["beta_threshold"], assign_by_max_beta=mode), 30, 100)
            extra["cfg5_condensates_ms_max_beta" if mode else "cfg5_condensates_ms_min_dist"] = round(m5[0], 3)
        # PushKnn forward / gradient over the cfg4 neighbour table (F=128)
        from hgcalml_amd import PushKnn
        pf = event_ms(lambda: torch.ops.hgcalml.push_knn(w4, x4, i4), 5, 2)
        pg = event_ms(lambda: torch.ops.hgcalml.push_knn_grad(g4[:, :F4].contiguous(), w4, x4, i4), 5, 2)
        extra["cfg4_push_knn_fwd_ms"], extra["cfg4_push_knn_grad_ms"] = round(pf[0], 3), round(pg[0], 3)
        # one GravNet block (learned 4-D coordinates -> kNN K=64+self -> accumulate F=64 -> dense), forward + backward
        from hgcalml_amd import RaggedGravNet
        torch.manual_seed(0)
        layer = RaggedGravNet(64, 64, 4, 128, 64, n_knn_bins=30).to(dev)
        xg = torch.from_numpy(c2["features"]).to(dev).requires_grad_(True)
        rs2 = torch.from_numpy(c2["row_splits"]).to(dev)

        def gravnet_step():
            out, _, _, dist = layer(xg, rs2)
            (out.sum() + dist.sum()).backward()
            xg.grad = None
        mg = event_ms(gravnet_step, 20, 40)
        extra["gravnet_block_fwd_bwd_ms_N150k_K64_F64"] = round(mg[0], 3)
    except Exception as e:  # information only; never hide the headline numbers
        extra["info_error"] = repr(e)

    # ------------------------------------------------------------------ CPU baseline
    cpu = None
    if not args.skip_cpu_baseline:
        log("bench: CPU baseline (oracle, 1 thread): binned kNN kernel over cfg2 ...")
        qps, secs = cpu_baseline_knn(c2)
        try:
            qps_o0, _ = cpu_baseline_knn(c2, reps=1, opt_level_0=True)
        except Exception as e:  # no compiler on this box and no prebuilt -O0 library
            log("bench: -O0 oracle unavailable (%r)" % (e,))
            qps_o0 = None
        small = workloads.cfg4(scale=0.1)
        f_s, b_s = cpu_baseline_accumulate(small)
        ns = len(small["indices"])
        import oracle
        c5_cpu = workloads.cfg5(ragged=True)
        t_c = time.perf_counter()
        oracle.BuildAndAssignCondensatesBinned(c5_cpu["ccoords"], c5_cpu["betas"], c5_cpu["dist"], c5_cpu["row_splits"],
                                               c5_cpu["beta_threshold"], assign_by_max_beta=True)
        cond_s = time.perf_counter() - t_c
        cpu = {"value": round(qps, 1), "unit": "queries/s", "cores": 1, "kind": "port",
               "sample": "5 passes over all %d queries of cfg2 through the oracle's binned_select_knn kernel "
                         "(gcc -O2, %.1f s); binning/sort glue not included" % (n2, secs),
               "accumulate_fwd_grad_GBps": round((4.0 * ns * (2 * K4 + 4 * F4) + 4.0 * ns * (3 * K4 + 5 * F4)) /
                                                 (f_s + b_s) / 1e9, 4),
               "accumulate_sample": "cfg4 at N=%d (fwd %.2f s, grad %.2f s)" % (ns, f_s, b_s),
               "condensates_cfg5_ms": round(cond_s * 1e3, 1),
               "condensates_sample": "all of cfg5 (8 uneven events, 500k hits, max-beta mode) through the oracle's wrapper "
                                     "(numpy glue + C kernel)",
               "value_unoptimised_build": None if qps_o0 is None else round(qps_o0, 1),
               "unoptimised_note": "same kernel built -O0 (the reference's Makefile passes no -O flag), one pass",
               "host_cpus": os.cpu_count(), "cpu_model": cpu_model()}
        log("bench: CPU oracle kNN %.0f queries/s (%.1f s)" % (qps, secs))

    traffic = measured_traffic() if args.roofline_scale == 1.0 else None
    valu_floor = measured_valu_floor() if args.roofline_scale == 1.0 else None
    floors_ms = [push_ms[0]] + ([valu_floor["ms"]] if valu_floor else [])
    with_build = (bytes_fwd + bytes_bwd) / ((fwd_ms[0] + grad_ms[0] + inv_ms[0]) * 1e-3) / 1e9
    line = {
        "metric": "kNN queries/s at N=150k,4D,K=64; accumulate_knn fwd+grad achieved HBM GB/s",
        "value": round(value, 1),
        "unit": "queries/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "cfg2: one event, N=150000 hits, 4-D clusters+noise, BinnedSelectKnn K=64 "
                               "(called with n_bins=30; the search runs on the library's own grid) + "
                               "AccumulateKnn(10 d^2) forward F=64",
                   "launch": launch_mode, "eager_ms_per_step": round(eager_ms_per_step, 4),
                   "knn_op_ms": round(knn_ms[0], 4), "accumulate_fwd_ms": round(acc2_ms[0], 4)},
        "accumulate_fwd_grad_GBps": round(achieved, 1),
        # the dominant kernel of the graded path: one launch of the one-pass gradient kernel
        "roofline": {"bound": "hbm",
                     "kernel": "hit_records_kernel + accumulate_grad_records_kernel + weight_grad_to_table_kernel: one "
                               "call of the accumulate_knn gradient (weights + features), cfg4 (N=%d, K=%d, F=%d)"
                               % (n4, K4, F4),
                     "achieved": round(bytes_bwd / (grad_ms[0] * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(bytes_bwd / (grad_ms[0] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                     "traffic": traffic["gradient"] if traffic else None,
                     "traffic_measured_at": traffic["measured_at"] if traffic else None,
                     "algorithmic_bytes": bytes_bwd, "launch_ms": round(grad_ms[0], 4),
                     # the same call through the gather that compares slot bytes (one kernel, no records)
                     "launch_ms_slot_byte_gather": round(grad_slots_ms[0], 4),
                     # floors of this formulation on this memory system: the bare K-fold gather of the same rows
                     # (PushKnn, timed above), the issue time of the gradient's vector instructions (counters)
                     "l2_gather_floor_ms": round(push_ms[0], 4),
                     "valu_floor_ms": valu_floor["ms"] if valu_floor else None,
                     "valu_floor_from": "profiles/accumulate_knn_cfg4_sq_tcc_counters.txt @ %s" %
                                        valu_floor["measured_at"] if valu_floor else None,
                     "frac_of_achievable": round(max(floors_ms) / grad_ms[0], 4),
                     "forward": {"kernel": "accumulate_fwd_wave_kernel, same workload, one launch",
                                 "achieved": round(bytes_fwd / (fwd_ms[0] * 1e-3) / 1e9, 1),
                                 "frac": round(bytes_fwd / (fwd_ms[0] * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                                 "traffic": traffic["forward"] if traffic else None,
                                 "algorithmic_bytes": bytes_fwd, "launch_ms": round(fwd_ms[0], 4)},
                     "forward_plus_gradient": {"achieved": round(achieved, 1), "frac": round(achieved / HBM_PEAK_GBS, 4),
                                               "algorithmic_bytes": bytes_fwd + bytes_bwd,
                                               "traffic": traffic["forward"] + traffic["gradient"] if traffic else None},
                     # the inverse neighbour index is rebuilt once per neighbour table, i.e. once per layer and
                     # training step: the pair with one build next to it
                     "forward_plus_gradient_with_index_build": {
                         "achieved": round(with_build, 1), "frac": round(with_build / HBM_PEAK_GBS, 4),
                         "ms": round(fwd_ms[0] + grad_ms[0] + inv_ms[0], 4)},
                     "inverse_index_build_ms": round(inv_ms[0], 3)},
        "cpu_baseline": cpu,
        "extra": extra,
    }
    if cpu:
        line["speedup_vs_cpu_kernel"] = round(n2 / (knn_ms[0] * 1e-3) / cpu["value"], 1)
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
