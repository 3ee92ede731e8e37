#!/usr/bin/env python3
"""Mini-batch construction benchmark on one MI355X.

A step is one mini-batch: multi-hop uniform neighbour sampling without
replacement + relabel on every hop + feature gather of the input nodes, with
the graph, the feature table and the seeds resident in HBM.  K steps are timed
back to back on one stream.  Prints ONE JSON line: sampled edges/s for the
whole step, the gather kernel's achieved HBM bandwidth against the 8 TB/s peak
(roofline, from HIP events carried by every gather dispatch of the timed region),
and the CPU oracle timed on this machine's host cores on a bounded sample of
the same workload (cpu_baseline).  stages.in_flight is the same K batches with
several batches in flight on separate streams.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload full|medium|small]
"""
import argparse
import ctypes
import json
import os
import sys
import time

HBM_PEAK_GBPS = 8000.0
# HBM bytes the gather kernel moves per gathered row, from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE runs of
# this script, each scaled by what the same counter reads for the plain copy kernel.  Keyed by everything the
# figure depends on, (workload, feature dtype, feature dim, batch); a run with any other combination reports
# traffic null.  Each entry names the profiles/ file that holds the counter readings.
MEASURED_GATHER_TRAFFIC_PER_ROW = {
    ("full", "bf16", 128, 4096): (520.2, "profiles/gather_kernel_full_pmc.txt"),           # (190.7 MB + 184.7 MB) / 721651 rows
    ("target", "bf16", 128, 1024): (519.0, "profiles/gather_kernel_target_bf16_pmc.txt"),  # (61.8 MB + 59.8 MB) / 234193 rows
    ("target", "fp32", 128, 1024): (1029.8, "profiles/gather_kernel_target_fp32_pmc.txt"),
    ("medium", "fp32", 100, 1024): (917.3, "profiles/gather_kernel_medium_pmc.txt"),       # 400-byte rows straddle lines
}

WORKLOADS = {
    # full-scale single GPU: 111M nodes, 3.2B directed edges, 128 x bf16, batch 4096
    "full": dict(nodes=111_059_956, edges=3_200_000_000, dim=128, dtype="bf16", batch=4096,
                 fan_out=[15, 10, 5]),
    # the same graph and features at batch 1024 (the shape the 60 %-of-peak gather target is stated on)
    "target": dict(nodes=111_059_956, edges=3_200_000_000, dim=128, dtype="bf16", batch=1024,
                   fan_out=[15, 10, 5]),
    # products-sized: 2.4M nodes, 62M edges, 100 x fp32, batch 1024
    "medium": dict(nodes=2_449_029, edges=62_000_000, dim=100, dtype="fp32", batch=1024,
                   fan_out=[15, 10, 5]),
    # one GPU's share of the full graph: a contiguous 1/8 of the rows, local features plus a
    # cache of the 20% hottest remote rows, misses bucketed into 8 owner request lists
    "partition": dict(nodes=111_059_956, edges=3_200_000_000, dim=128, dtype="fp32", batch=1024,
                      fan_out=[15, 10, 5], parts=8, part=3, cache_ratio=0.2),
    # the small plumbing case: 100k nodes, 2 hops
    "small": dict(nodes=100_000, edges=1_500_000, dim=128, dtype="fp32", batch=1024, fan_out=[10, 5]),
}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="full", choices=sorted(WORKLOADS))
    ap.add_argument("--batch_size", type=int, default=None)
    ap.add_argument("--feature_dtype", default=None, choices=["fp32", "bf16"])
    ap.add_argument("--fan_out", type=str, default=None,
                    help="comma list, k-hop..1-hop as in the reference (the seeds use the last entry)")
    ap.add_argument("--replace", action="store_true", help="sample with replacement (reference semantics)")
    ap.add_argument("--cpu_seconds", type=float, default=12.0,
                    help="seconds of CPU-oracle work for the cpu_baseline leg (0 = skip)")
    ap.add_argument("--cpu_threads", type=int, default=None)
    ap.add_argument("--seed", type=int, default=1)
    ap.add_argument("--driver", default="fused", choices=["graph", "fused", "unfused"],
                    help="graph: fused C driver replayed as a HIP graph; fused: same, launched eagerly; "
                         "unfused: per-hop sample + hash relabel calls")
    ap.add_argument("--inflight", type=int, default=4,
                    help="after the timed single-stream region, also run the K batches with N of them in "
                         "flight (N pipelines on N HIP streams) and report it under stages.in_flight; 1 = skip")
    ap.add_argument("--calibration_copy_mib", type=int, default=0,
                    help="also launch the plain copy kernel once on this many MiB (for scaling "
                         "FETCH_SIZE / WRITE_SIZE when the run is under rocprofv3 --pmc)")
    ap.add_argument("--formats", action="store_true",
                    help="also time the emission of every hop's block as COO + CSC (+ CSR)")
    ap.add_argument("--aggregation", action="store_true",
                    help="also time GraphSAGE-style SpMM (hidden 256, fp32 and bf16) and SDDMM on the "
                         "outermost sampled block of the last batch")
    ap.add_argument("--shuffle", action="store_true",
                    help="also time the local halves of the feature shuffle on the batch's input nodes: bucketing by "
                         "owner (cluster_permute) and pack / unpack of hidden rows")
    ap.add_argument("--cache_build", action="store_true",
                    help="also time the cache-construction kernels (access counting, cached CSR of the hottest rows, "
                         "cached feature table) and one step of the all-strategies dry run")
    ap.add_argument("--gather_sizes", action="store_true",
                    help="also time the gather kernel alone on 0 .. 940 k random rows of this workload's table "
                         "(device-side count, every launch with its own events): what a launch costs before it moves a byte")
    ap.add_argument("--frontier_order", action="store_true",
                    help="also time the last hop's sampling on the frontier in first-occurrence order (as the relabel "
                         "leaves it) and in node-id order")
    ap.add_argument("--phase_costs", action="store_true",
                    help="also measure what separates two dependent phases: a launch boundary (chain of empty kernels) "
                         "against a grid-wide barrier inside one kernel of 32..256 co-resident workgroups")
    ap.add_argument("--relabel_small", action="store_true",
                    help="also time apt_relabel on first-hop-sized inputs: one workgroup with the table in LDS "
                         "against the passes over a table in device memory")
    ap.add_argument("--tune", type=str, default="", help="kernel-variant knobs, e.g. sample_lanes_per_row=16")
    ap.add_argument("--target_leg", default="auto", choices=["auto", "on", "off"],
                    help="after the timed region also run batch 1024 on the same graph with 128 x bf16 and 128 x fp32 "
                         "features (the shape the 60 %%-of-peak gather target is stated on) and report it under "
                         "stages.target_shape; auto = only for workload full")
    ap.add_argument("--target_steps", type=int, default=100)
    ap.add_argument("--event_steps", type=int, default=32,
                    help="how many (evenly spaced) steps of the timed region carry kernel events")
    ap.add_argument("--ceilings", default="auto", choices=["auto", "on", "off"],
                    help="measure the GPU's rate for random 4-byte loads / stores / atomics (what bounds the sampling "
                         "kernel) and quote the last hop's sampling kernel against it; auto = on")
    ap.add_argument("--defer_lookup", default="off", choices=["on", "off"],
                    help="on: the relabel's last pass rides in the gather's launch instead of being a launch of its "
                         "own before it (MiniBatchPipeline(defer_lookup=True)); the default run reports the batch "
                         "time that way under stages.deferred_lookup")
    ap.add_argument("--alternate", type=str, default="",
                    help="settings to compare inside this one process, separated by '/', each a '+'-joined list of "
                         "knob=value (e.g. gather_wt_tail_mib=1/gather_wt_tail_mib=64): the batches of the timed region "
                         "are run again and again with the settings taking turns (stages.alternate); two processes, "
                         "let alone two boxes, differ by more than most knobs do")
    ap.add_argument("--alternate_batch", type=int, default=0, help="batch size of --alternate (0 = the workload's)")
    ap.add_argument("--ceiling_table_mib", type=str, default="",
                    help="comma-separated table sizes in MiB: repeat the random-access measurement for each "
                         "(stages.random_access_by_table_size)")
    return ap.parse_args()

def quantiles(xs):
    """median / p10 / p90 / min / max of a list (nearest rank)."""
    v = sorted(xs)
    at = lambda q: v[min(len(v) - 1, max(0, int(round(q * (len(v) - 1)))))]
    return {"median": at(0.5), "p10": at(0.1), "p90": at(0.9), "min": v[0], "max": v[-1], "n": len(v)}


class KernelEvents:
    """Pairs of HIP events that ride on a kernel dispatch (kernel begin / kernel end), see
    apt_time_next_gather / apt_time_next_sample."""

    def __init__(self):
        self.hip = ctypes.CDLL("libamdhip64.so")
        self.hip.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        self.hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
        self.hip.hipEventDestroy.argtypes = [ctypes.c_void_p]

    def pair(self):
        a, b = ctypes.c_void_p(), ctypes.c_void_p()
        assert self.hip.hipEventCreate(ctypes.byref(a)) == 0 and self.hip.hipEventCreate(ctypes.byref(b)) == 0
        return a, b

    def ms(self, pair, destroy=True):
        ms = ctypes.c_float()
        rc = self.hip.hipEventElapsedTime(ctypes.byref(ms), pair[0], pair[1])
        assert rc == 0, f"hipEventElapsedTime -> {rc}"
        if destroy:
            self.hip.hipEventDestroy(pair[0])
            self.hip.hipEventDestroy(pair[1])
        return ms.value


def gather_bytes_per_row(dim, esize, has_pos_map):
    """-> (bytes the launch moves per row, the per-row figure of the roofline definition).  Row read + row
    write + 8-byte id (+ the 8-byte position-map entry: the definition always counts it, the launch only reads
    it when the store has a map; an identity store has none)."""
    return 2 * dim * esize + 8 + (8 if has_pos_map else 0), 2 * dim * esize + 16


def stage_target_shape(args, capi, dev, graph, hops, kev, MiniBatchPipeline, N, seed_n, store_of, synth, torch):
    """Batch 1024 on the same graph with 128 x bf16 and 128 x fp32 rows: the shape the gather target
    (>= 60 % of HBM peak) is stated on.  Every gather dispatch carries events; the sizes of every batch are
    kept on the device and read afterwards, so each launch's rows and duration give its own fraction.
    The figures are of the gather kernel launched by itself (the relabel's last pass as a launch of its own
    before it); the pipeline's default lets that pass ride in the gather's launch, which makes the batch
    shorter and that launch a little longer: `with_lookup_riding` has the same batches that way."""
    B, Kt, Wt, H = 1024, args.target_steps, 20, len(hops)
    gen = torch.Generator(device=dev)
    gen.manual_seed(args.seed + 77)
    out = {"batch": B, "batches": Kt, "warmup": Wt}
    for name in ("bf16", "fp32"):
        store = store_of(name)
        esize = store.local_table.element_size()
        moved, spec = gather_bytes_per_row(store.out_dim, esize, store.pos_map is not None)
        pipe = MiniBatchPipeline(graph, store, B, hops, replace=args.replace, fused=args.driver != "unfused",
                                 defer_lookup=args.defer_lookup == "on")
        pool = torch.randperm(seed_n, generator=gen, device=dev)[:(Kt + Wt) * B]
        sets = [pool[i * B:(i + 1) * B].contiguous() for i in range(Kt + Wt)]
        del pool
        log = torch.zeros((Kt, H + 2), dtype=torch.int64, device=dev)
        for i in range(Wt):
            pipe.run(sets[i], args.seed + 5000 + i)
        torch.cuda.synchronize()

        def timed_pass(defer):
            pairs = []
            step_ev = [torch.cuda.Event(enable_timing=True) for _ in range(Kt + 1)]
            step_ev[0].record()
            for i in range(Kt):
                pipe.sample(sets[Wt + i], args.seed + 5000 + Wt + i, defer_lookup=defer)
                pairs.append(kev.pair())
                capi.check(capi.lib().apt_time_next_gather(*pairs[-1]))
                pipe.gather()
                log[i].copy_(pipe.sizes)
                step_ev[i + 1].record()
            torch.cuda.synchronize()
            assert int(pipe.misses.item()) == 0
            us = [kev.ms(pr) * 1e3 for pr in pairs]
            rows = log[:, H].cpu().tolist()
            frac = [r * moved / (t * 1e-6) / 1e9 / HBM_PEAK_GBPS for r, t in zip(rows, us)]
            return us, rows, frac, [step_ev[i].elapsed_time(step_ev[i + 1]) for i in range(Kt)]

        def wall_pass(defer):
            """The same batches back to back without events or size copies: wall time per batch."""
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for i in range(Kt):
                pipe.sample(sets[Wt + i], args.seed + 5000 + Wt + i, defer_lookup=defer)
                pipe.gather()
            torch.cuda.synchronize()
            return (time.perf_counter() - t0) / Kt

        us, rows, frac, step_ms = timed_pass(False)
        edges = log[:, H + 1].cpu().tolist()
        wall_alone = wall_pass(False)
        riding = None
        if pipe.can_defer_lookup:
            us_r, _, frac_r, _ = timed_pass(True)
            riding = {"us_median": quantiles(us_r)["median"], "frac": quantiles(frac_r)["median"],
                      "frac_p10": quantiles(frac_r)["p10"], "ms_per_step": wall_pass(True) * 1e3}
        wall = riding["ms_per_step"] * 1e-3 if riding else wall_alone     # what a pipeline does by default
        q_us, q_frac = quantiles(us), quantiles(frac)
        out[name] = {
            "rows": sum(rows) / Kt, "bytes_per_row": moved, "bytes_per_row_definition": spec,
            "us_median": q_us["median"], "us_p10": q_us["p10"], "us_p90": q_us["p90"], "us_min": q_us["min"],
            "us_max": q_us["max"],
            # fraction of 8 TB/s of each launch (its own rows over its own duration); p10 = the slow end
            "frac": q_frac["median"], "frac_p10": q_frac["p10"], "frac_p90": q_frac["p90"],
            "frac_min": q_frac["min"], "frac_max": q_frac["max"],
            "frac_by_definition_bytes": q_frac["median"] * spec / moved,
            "traffic_bytes_per_row": MEASURED_GATHER_TRAFFIC_PER_ROW.get(("target", name, store.out_dim, B), (None, None))[0],
            "traffic_source": MEASURED_GATHER_TRAFFIC_PER_ROW.get(("target", name, store.out_dim, B), (None, None))[1],
            "GBps_median": q_frac["median"] * HBM_PEAK_GBPS,
            "ms_per_step": wall * 1e3, "ms_per_step_gather_launched_alone": wall_alone * 1e3,
            "ms_per_step_events": quantiles(step_ms),
            "edges_per_s": sum(edges) / Kt / wall,
            "with_lookup_riding": riding,
        }
        del pipe, log, sets
    return out


def graph_replay_us(torch, fn, reps=10, replays=5):
    """us per call of fn(): `reps` calls captured into a HIP graph on a side stream and replayed, so that
    the host's share of a call is not in the figure."""
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=torch.cuda.Stream()):
        for _ in range(reps):
            fn()
    g.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(replays):
        g.replay()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / (replays * reps) * 1e3


def stage_gather_sizes(capi, dev, kev, store, N, torch):
    """The gather kernel alone on n random rows (distinct ids per launch, so the memory-side cache serves
    nothing twice), device-side count under a host bound of 1 081 344 rows (what batch 1024 allocates): the
    duration of a launch that gathers nothing is what every launch pays before it moves a byte."""
    cap = 1024 * 6 * 11 * 16
    gen = torch.Generator(device=dev)
    gen.manual_seed(5)
    pool = torch.randperm(N, generator=gen, device=dev)[:cap * 8].contiguous()
    out = torch.empty((cap, store.out_dim), dtype=store.dtype, device=dev)
    esize = store.local_table.element_size()
    moved, _ = gather_bytes_per_row(store.out_dim, esize, store.pos_map is not None)
    rows = []
    for n in (0, 1024, 16384, 65536, 131072, 235000, 470000, 940000):
        n_dev = torch.tensor([n], dtype=torch.int64, device=dev)
        us = []
        for rep in range(45):
            off = (rep * 917519) % (pool.numel() - cap)
            pr = kev.pair()
            capi.check(capi.lib().apt_time_next_gather(*pr))
            capi.gather_rows(store, pool[off:off + cap], num_index_dev=n_dev, out=out)
            torch.cuda.synchronize()
            t = kev.ms(pr) * 1e3
            if rep >= 5:
                us.append(t)
        q = quantiles(us)
        rows.append({"rows": n, "us_min": q["min"], "us_median": q["median"], "us_p90": q["p90"],
                     "GBps_median": n * moved / q["median"] / 1e3,
                     # the kernel's own rule: write-through stores while the output is at most 128 MB
                     "stores": "write-through" if n * store.out_dim * esize <= (128 << 20) else "non-temporal"})
    del pool, out
    # least-squares line through the medians of the write-through launches that move data: us = fixed + bytes / rate
    pts = [(r["rows"] * moved / 1e6, r["us_median"]) for r in rows if r["rows"] >= 16384 and r["stores"] == "write-through"]
    mx = sum(x for x, _ in pts) / len(pts)
    my = sum(y for _, y in pts) / len(pts)
    slope = sum((x - mx) * (y - my) for x, y in pts) / sum((x - mx) ** 2 for x, _ in pts)
    return {"bytes_per_row": moved, "launches": rows,
            "fit_write_through_launches_from_16k_rows": {"fixed_us": my - slope * mx, "streaming_GBps": 1e3 / slope}}


def stage_frontier_order(args, capi, dev, graph, hops, seed_sets, stage_pipe, torch, W):
    """The last hop's sampling (no relabel marking) on its frontier as the relabel leaves it and in node-id order."""
    H = len(hops)
    stage_pipe.sample(seed_sets[W], args.seed + 100 + W)
    torch.cuda.synchronize()
    n = int(stage_pipe.sizes[H - 1].item())
    front = stage_pipe.nodes[:n].clone()
    srt = torch.sort(front).values.contiguous()
    f = hops[-1]
    out = torch.empty(n * f, dtype=torch.int64, device=dev)
    cnt = torch.empty(n, dtype=torch.int64, device=dev)
    res = {"rows": n, "fanout": f}
    for name, fr in (("first_occurrence_order_us", front), ("node_id_order_us", srt)):
        res[name] = graph_replay_us(torch, lambda: capi.sample_neighbors(graph, fr, f, args.replace, 7, H - 1,
                                                                         out_neighbors=out, out_counts=cnt))
    del front, srt, out, cnt
    return res


def stage_phase_costs(capi, dev, torch):
    """A launch boundary against a grid-wide barrier (us per dependent phase)."""
    L = capi.lib()
    buf = torch.zeros(1024 * 256, dtype=torch.int32, device=dev)
    state = torch.zeros(192, dtype=torch.int32, device=dev)

    def best_ms(fn, reps=6):
        best = None
        for _ in range(reps):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            fn()
            e1.record()
            torch.cuda.synchronize()
            t = e0.elapsed_time(e1)
            best = t if best is None or t < best else best
        return best

    launches = lambda n: capi.check(L.apt_synth_empty_launches(n, capi._ptr(buf), capi._stream()))
    res = {"dependent_empty_launch_us": (best_ms(lambda: launches(44)) - best_ms(lambda: launches(4))) / 40 * 1e3,
           "grid_barrier_us_per_phase": {}}
    for groups in (32, 64, 128, 256):
        run = lambda ph: capi.check(L.apt_synth_grid_barrier(groups, ph, capi._ptr(state), capi._ptr(buf), capi._stream()))
        res["grid_barrier_us_per_phase"][str(groups)] = (best_ms(lambda: run(44)) - best_ms(lambda: run(4))) / 40 * 1e3
    res["barrier_failures"] = int(state[128].item())
    return res


def stage_relabel_small(capi, dev, N, torch):
    """apt_relabel on inputs the size of a batch's first hop: the single-workgroup LDS kernel against the five
    passes over a table in device memory (relabel_lds switched off).  Twenty calls are captured into a HIP
    graph and replayed, so the host's share of a call is not in the figure."""
    gen = torch.Generator(device=dev)
    gen.manual_seed(11)

    out = []
    for ns, f in ((256, 15), (1024, 5), (512, 10), (1024, 7)):
        seeds = torch.randperm(N, generator=gen, device=dev)[:ns].contiguous()
        nbrs = torch.randint(0, N, (ns * f,), generator=gen, device=dev)
        nbrs[::3] = seeds[torch.randint(0, ns, (nbrs[::3].numel(),), generator=gen, device=dev)]   # repeats of the seeds
        uniq = torch.empty(ns * (f + 1), dtype=torch.int64, device=dev)
        rel = torch.empty(ns * f, dtype=torch.int64, device=dev)
        cnt = torch.empty(1, dtype=torch.int64, device=dev)
        ws = torch.empty(capi.relabel_workspace_bytes(ns * (f + 1)), dtype=torch.uint8, device=dev)
        row = {"seeds": ns, "fanout": f, "items": ns * (f + 1)}
        for key, lds in (("lds_one_launch_us", 1), ("device_table_five_launches_us", 0)):
            capi.set_tuning("relabel_lds", lds)
            row[key] = graph_replay_us(torch, lambda: capi.relabel(seeds, nbrs, unique=uniq, relabeled=rel,
                                                                   num_unique_dev=cnt, workspace=ws, sync=False), reps=20)
        capi.set_tuning("relabel_lds", 1)
        out.append(row)
    return out


def stage_alternate(args, capi, graph, hops, kev, MiniBatchPipeline, seed_n, seed_lo, store, B, torch, dev):
    """Kernel-variant knobs against each other inside one process: six rounds, in each of which every setting
    runs the same 35 batches on one stream (wall time) and 20 more whose gather and last-hop sampling dispatches
    carry events.  The first five batches after a change of setting still run behind the previous setting's
    gather and are left out.  -> per setting: medians over the rounds."""
    import statistics as st
    settings = []
    for text in args.alternate.split("/"):
        knobs = dict((kv.split("=")[0], int(kv.split("=")[1])) for kv in text.split("+"))
        settings.append((text, knobs))
    touched = sorted({k for _, knobs in settings for k in knobs})
    default_of = lambda k: 1 if k in ("minibatch_fuse_mark", "relabel_lds", "block_fused_scan") else 0
    H, NB = len(hops), 40
    pipe = MiniBatchPipeline(graph, store, B, hops, replace=args.replace, fused=args.driver != "unfused")
    gen = torch.Generator(device=dev)
    gen.manual_seed(args.seed + 31)
    pool = seed_lo + torch.randperm(seed_n, generator=gen, device=dev)[:NB * B]
    sets = [pool[i * B:(i + 1) * B].contiguous() for i in range(NB)]
    res = {text: {"ms": [], "gather_us": [], "sample_us": []} for text, _ in settings}
    for i in range(NB):
        pipe.run(sets[i], args.seed + 900 + i)
    torch.cuda.synchronize()
    try:
        for rnd in range(7):
            for text, knobs in settings:
                for k in touched:
                    capi.set_tuning(k, knobs.get(k, default_of(k)))
                for i in range(5):
                    pipe.run(sets[i], args.seed + 900 + i)
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for i in range(5, NB):
                    pipe.run(sets[i], args.seed + 900 + i)
                torch.cuda.synchronize()
                ms = (time.perf_counter() - t0) / (NB - 5) * 1e3
                gp, sp = [], []
                for i in range(5, 25):
                    g, s = kev.pair(), kev.pair()
                    if args.driver == "fused":
                        capi.check(capi.lib().apt_time_next_sample(H - 1, s[0], s[1]))
                    pipe.sample(sets[i], args.seed + 900 + i, defer_lookup=True)
                    capi.check(capi.lib().apt_time_next_gather(g[0], g[1]))
                    pipe.gather()
                    gp.append(g)
                    sp.append(s)
                torch.cuda.synchronize()
                g_us = st.median(kev.ms(p) * 1e3 for p in gp)
                s_us = st.median(kev.ms(p) * 1e3 for p in sp) if args.driver == "fused" else None
                if rnd > 0:   # the first round warms up
                    res[text]["ms"].append(ms)
                    res[text]["gather_us"].append(g_us)
                    res[text]["sample_us"].append(s_us)
    finally:
        for k in touched:
            capi.set_tuning(k, default_of(k))
        for kv in filter(None, args.tune.split(",")):
            capi.set_tuning(kv.split("=")[0], int(kv.split("=")[1]))
    out = {"batch": B, "rounds": 6, "batches_per_round": NB - 5, "settings": []}
    for text, _ in settings:
        r = res[text]
        out["settings"].append({
            "setting": text, "ms_per_batch_median": st.median(r["ms"]), "ms_per_batch_by_round": r["ms"],
            "gather_us_median": st.median(r["gather_us"]),
            "last_hop_sample_us_median": st.median(r["sample_us"]) if args.driver == "fused" else None})
    return out


def stage_ceilings(capi, dev, N, torch, table_bytes=None):
    """The GPU's rate for one random 4-byte access per work item into a table of the rank table's size
    (or of table_bytes)."""
    nbytes = table_bytes if table_bytes else max(1 << 20, (N * 4 + 15) // 16 * 16)
    table = torch.full((nbytes // 4,), -1, dtype=torch.int32, device=dev)
    sink = torch.zeros(1, dtype=torch.int32, device=dev)
    n = 8_000_000
    res = {"table_bytes": nbytes, "accesses_per_launch": n}
    for mode, name in ((0, "load"), (1, "store"), (2, "atomic_min"), (3, "atomic_min_returning"), (4, "load_16B"),
                       (5, "load_and_atomic_min_pairs")):
        ts = []
        for rep in range(7):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            capi.check(capi.lib().apt_synth_random_access(mode, capi._ptr(table), nbytes, n, rep + 1,
                                                          capi._ptr(sink), capi._stream()))
            e1.record()
            torch.cuda.synchronize()
            if rep >= 2:
                ts.append(e0.elapsed_time(e1) * 1e-3)
        ts.sort()
        res[name + "_G_per_s"] = n / ts[len(ts) // 2] / 1e9
    del table, sink
    return res


def seconds_per_call(torch, fn, reps=10, warm=3):
    """Mean duration of fn() on the current stream: `reps` back-to-back calls between two events."""
    for _ in range(warm):
        fn()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / reps * 1e-3


def stage_aggregation(args, capi, dev, K, seed_sets, stage_pipe, synth, torch, W):
    """Optional aggregation stage on the outermost block of the last batch."""
    stage_pipe.run(seed_sets[W + K - 1], args.seed + 100 + W + K - 1)
    res = stage_pipe.result()
    blk = res["blocks"][0]
    rel = blk["relabeled"]
    f = blk["fanout"]
    col_all = torch.arange(blk["seeds"].numel(), device=dev).repeat_interleave(f)
    keep = rel >= 0
    row_e, col_e = rel[keep].contiguous(), col_all[keep].contiguous()
    n_src, n_dst, E, hid = blk["unique"].numel(), blk["seeds"].numel(), int(keep.sum()), 256
    agg = {"edges": E, "num_src": n_src, "num_dst": n_dst, "hidden": hid}
    for name, dt, es in (("fp32", torch.float32, 4), ("bf16", torch.bfloat16, 2)):
        h = synth.random_features(n_src, hid, dt, args.seed + 7, dev)
        fn = lambda: capi.spmm_sum(0, row_e, col_e, h, n_dst)
        t = seconds_per_call(torch, fn)
        nbytes = E * hid * es + 2 * n_dst * hid * 4 + 16 * E   # rows read, zero-fill + sums written, ids
        agg[f"spmm_copy_u_sum_{name}_us"] = t * 1e6
        agg[f"spmm_copy_u_sum_{name}_GBps"] = nbytes / t / 1e9
        # the same sum (as a mean) straight from the sampler's fixed-stride block layout
        fn = lambda: capi.spmm_block(rel, n_dst, f, h, mean=True)
        t = seconds_per_call(torch, fn)
        nbytes = E * hid * es + n_dst * hid * 4 + 8 * n_dst * f
        agg[f"spmm_block_mean_{name}_us"] = t * 1e6
        agg[f"spmm_block_mean_{name}_GBps"] = nbytes / t / 1e9
    # GAT layer of the same block: 4 heads x 64, logits then fused LeakyReLU + edge softmax + weighted sum
    heads, hdim = 4, 64
    for name, dt, es in (("fp32", torch.float32, 4), ("bf16", torch.bfloat16, 2)):
        ft = synth.random_features(n_src, heads * hdim, dt, args.seed + 9, dev).view(n_src, heads, hdim)
        al = (torch.randn(heads, hdim, device=dev) * 0.02).contiguous()
        ar = (torch.randn(heads, hdim, device=dev) * 0.02).contiguous()
        el, er = capi.gat_scores(ft, al), capi.gat_scores(ft[:n_dst], ar)
        for tag, fn, nbytes in (
                ("gat_scores", lambda: capi.gat_scores(ft, al), n_src * heads * (hdim * es + 4)),
                ("gat_block", lambda: capi.gat_block(rel, n_dst, f, ft, el, er, 0.2),
                 E * heads * (hdim * es + 4) + n_dst * heads * (hdim * 4 + 4) + 8 * n_dst * f)):
            t = seconds_per_call(torch, fn)
            agg[f"{tag}_{name}_us"] = t * 1e6
            agg[f"{tag}_{name}_GBps"] = nbytes / t / 1e9
        # backward of the aggregation: logit gradients per (destination, head), then the sums over the
        # edges of a source on the block's CSR order
        fmt_b = capi.block_formats(rel, n_dst, f, n_src)
        _, attn_w = capi.gat_block(rel, n_dst, f, ft, el, er, 0.2, want_attn=True)
        d_out = torch.randn(n_dst, heads, hdim, device=dev)
        csr_ip = fmt_b["csr_indptr"][:n_src + 1].contiguous()
        src_csr = fmt_b["coo_row"][fmt_b["csr_eids"]].contiguous()
        d2 = d_out.view(n_dst, heads * hdim)

        def gat_bwd():
            a_e, dz_e, d_er = capi.gat_block_backward(rel, n_dst, f, ft, el, er, 0.2, attn_w, d_out,
                                                      fmt_b["csc_indptr"], fmt_b["num_edges"])
            capi.spmm_heads(fmt_b["csr_indices"], src_csr, d_out, a_e, n_src, weight_row=fmt_b["csr_eids"],
                            grouped=True, head_weights2=dz_e, out_indptr=csr_ip)

        # backward of the plain sum / mean (SAGE, GCN): the same sum over the CSR order, no weights
        for tag, fn in (("gat_block_backward", gat_bwd),
                        ("spmm_block_backward", lambda: capi.spmm_heads(
                            fmt_b["csr_indices"], src_csr, d2, None, n_src, grouped=True, out_indptr=csr_ip))):
            if tag.startswith("spmm_block_backward") and name != "fp32":
                continue
            agg[f"{tag}_{name}_us"] = seconds_per_call(torch, fn) * 1e6
        del ft, el, er, fmt_b, attn_w, d_out
    hd = synth.random_features(n_dst, hid, torch.float32, args.seed + 8, dev)
    h = synth.random_features(n_src, hid, torch.float32, args.seed + 7, dev)
    fn = lambda: capi.sddmm(0, row_e, col_e, h, hd)
    t = seconds_per_call(torch, fn)
    agg["sddmm_u_add_v_fp32_us"] = t * 1e6
    agg["sddmm_u_add_v_fp32_GBps"] = (3 * E * hid * 4 + 16 * E) / t / 1e9
    del h, hd
    return agg


def stage_formats(args, B, ev, graph, hops, K, MiniBatchPipeline, requests, seed_sets, store, torch, W):
    """Optional: every hop's block as COO + CSC (+ CSR), device-side sizes, after sampling."""
    fmt = {}
    for name, what in (("coo_csc", "csc"), ("coo_csc_csr", True)):
        fp = MiniBatchPipeline(graph, store, B, hops, replace=args.replace, formats=what, requests=requests)
        t = 0.0
        for i in range(W + K):
            m = (ev(), ev())
            fp.sample(seed_sets[i], args.seed + 100 + i)
            m[0].record()
            fp.emit_formats()
            m[1].record()
            torch.cuda.synchronize()
            if i >= W:
                t += m[0].elapsed_time(m[1])
        fmt[name + "_ms"] = t / K                       # the hops beside each other, nothing else running
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(K):
            fp.run(seed_sets[W + i], args.seed + 100 + W + i)
        torch.cuda.synchronize()
        fmt[name + "_whole_batch_ms"] = (time.perf_counter() - t0) / K * 1e3   # sampling + formats beside the gather
        del fp
    return fmt


def stage_shuffle(args, capi, dev, hops, N, seed_sets, stage_pipe, torch, W):
    """Optional: bucketing by owner and pack / unpack of hidden rows (the local halves of feat_shuffle)."""
    ms_of = lambda fn: seconds_per_call(torch, fn) * 1e3

    stage_pipe.run(seed_sets[W], args.seed + 100 + W)
    torch.cuda.synchronize()
    H = len(hops)
    n_in = int(stage_pipe.sizes[H].item())
    ids = stage_pipe.nodes[:n_in].contiguous()
    world, hid = 8, 256
    mv = torch.linspace(0, N, world + 1).to(torch.int64).to(dev)
    t_bucket = ms_of(lambda: capi.cluster_permute(ids, mv, world))
    _, _, _, perm = capi.cluster_permute(ids, mv, world)
    hrows = torch.randn(n_in, hid, device=dev)
    t_unpack = ms_of(lambda: capi.permute_rows(hrows, perm))
    t_pack = ms_of(lambda: capi.scatter_rows(hrows, perm))
    row_bytes = 2 * hid * 4 + 8
    shuffle = {"ids": n_in, "owners": world, "hidden": hid,
               "cluster_permute_us": t_bucket * 1e3, "cluster_permute_GBps": 24.0 * n_in / (t_bucket * 1e-3) / 1e9,
               "unpack_us": t_unpack * 1e3, "unpack_GBps": n_in * row_bytes / (t_unpack * 1e-3) / 1e9,
               "pack_us": t_pack * 1e3, "pack_GBps": n_in * row_bytes / (t_pack * 1e-3) / 1e9}
    del hrows, perm, ids
    return shuffle


def stage_cache_build(args, B, bytes_per_row, capi, dev, graph, hops, indptr, N, seed_sets, stage_pipe, store, torch,
                      W):
    """Optional: cache construction and the strategy dry run (the callers of the registries)."""
    from apt_amd import cache as cache_mod
    from apt_amd import cost_model as cm

    time_ms = lambda fn, reps=5: seconds_per_call(torch, fn, reps=reps, warm=1) * 1e3

    stage_pipe.run(seed_sets[W], args.seed + 100 + W)
    torch.cuda.synchronize()
    H = len(hops)
    n_in = int(stage_pipe.sizes[H].item())
    counter = cache_mod.HotnessCounter(N, dev)
    t_count = time_ms(lambda: counter.add(stage_pipe.nodes, n_dev=stage_pipe.sizes[H:H + 1], output_nodes=seed_sets[W]))
    deg = indptr[1:] - indptr[:-1]
    hot = torch.topk(deg, min(1_000_000, N // 4)).indices.contiguous()
    t_csr = time_ms(lambda: cache_mod.build_graph_cache(graph, hot), reps=3)
    c_edges = int(deg[hot].sum().item())
    t_feat = time_ms(lambda: capi.gather_rows(store, hot), reps=3)
    world = 8
    mv = torch.linspace(0, N, world + 1).to(torch.int64)
    run = cm.AllPSDryRun(graph, world, list(reversed(hops)), mv, rng_seed=args.seed)
    per_rank = [seed_sets[i % len(seed_sets)] for i in range(world)]
    run.sample(per_rank)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    res = run.sample(per_rank)
    torch.cuda.synchronize()
    t_dry = time.perf_counter() - t0
    cache_build = {
        "count_ids_us": t_count * 1e3, "count_ids_nodes": n_in + B,
        "cached_csr_rows": int(hot.numel()), "cached_csr_edges": c_edges, "cached_csr_ms": t_csr,
        "cached_csr_GBps": 16.0 * c_edges / (t_csr * 1e-3) / 1e9,          # every edge read and written once
        "cached_features_ms": t_feat, "cached_features_GBps": hot.numel() * bytes_per_row / (t_feat * 1e-3) / 1e9,
        "dry_run_all_strategies_ms_per_step": t_dry * 1e3, "dry_run_world_size": world,
        "dry_run_input_nodes_rank0": {"DP": int(res[0].dp_seeds.numel()), "NP": int(res[0].np_seeds.numel()),
                                      "SP": int(res[0].sp_seeds.numel()), "MP": int(res[0].mp_seeds.numel())},
    }
    del counter, hot, deg, run, res
    return cache_build


def stage_cpu_baseline(args, bytes_per_row, cache, dtype, feats, hops, indices, indptr, K, lo, min_vids, N, P, pos_map,
                       requests, seed_sets, torch, W):
    """CPU baseline: the oracle on this machine's host cores, bounded sample."""
    budget = args.cpu_seconds
    import numpy as np

    import oracle as orc
    threads = args.cpu_threads or min(16, orc.max_threads())
    orc.set_threads(threads)
    h_indptr = indptr.cpu().numpy()
    h_indices = indices.cpu().numpy()
    if dtype == torch.bfloat16:
        h_feats = feats.view(torch.int16).cpu().numpy().view(np.uint16)
    else:
        h_feats = feats.cpu().numpy()
    to_np = lambda t: (t.view(torch.int16).cpu().numpy().view(np.uint16) if t.dtype == torch.bfloat16
                       else t.cpu().numpy())
    if requests is None:
        og = orc.Graph(h_indptr, h_indices)
        ofs = orc.FeatStore(h_feats)
    else:
        h_pos = pos_map.cpu().numpy()
        og = orc.Graph(h_indptr, h_indices, row_begin=lo, num_total_nodes=N)
        ofs = orc.FeatStore(h_feats, to_np(cache), h_pos)
        h_mv, h_rw = min_vids.cpu().numpy(), requests["remote_worker_map"].cpu().numpy()
    h_seeds = [s.cpu().numpy() for s in seed_sets[W:]]
    def cpu_leg(seconds, first):
        """Batches of the timed seed sets (cycled with fresh rng keys) until `seconds` are used."""
        edges_done = batches = 0
        tc = 0.0
        while tc < seconds:
            s = h_seeds[(first + batches) % K]
            key = args.seed + 100 + W + first + batches
            t1 = time.perf_counter()
            inp, blocks = orc.sample_blocks(og, s, hops, args.replace, key)
            if requests is None:
                orc.gather_rows(ofs, inp)
            else:
                bs, _, so, _ = orc.cluster_reqs(inp, h_pos, h_rw, h_mv, P, P)
                orc.gather_rows(ofs, so[:bs[0]])
            tc += time.perf_counter() - t1
            edges_done += sum(int(b["counts"].sum()) for b in blocks)
            batches += 1
        return edges_done, batches, tc

    # most of the budget on all threads (the reported value), the rest on one thread for reference
    cpu_edges, cpu_batches, tc = cpu_leg(budget * 0.75, 0)
    one = None
    if threads > 1:
        orc.set_threads(1)
        e1, b1, t1s = cpu_leg(budget * 0.25, cpu_batches)
        one = dict(value=e1 / t1s, batches=b1, seconds=t1s)
        orc.set_threads(threads)
    # the gather stage alone, as the reference states it on the CPU (src/load_subtensor.cc:10-17: torch's
    # index_select over the host table), on the input nodes of one batch
    gather_cpu = None
    if requests is None:
        inp, _ = orc.sample_blocks(og, h_seeds[0], hops, args.replace, args.seed + 100 + W)
        table = torch.from_numpy(h_feats.view(np.int16) if dtype == torch.bfloat16 else h_feats)
        ids_t = torch.from_numpy(inp)
        torch.set_num_threads(threads)
        table.index_select(0, ids_t[:1000])
        t1 = time.perf_counter()
        reps = 0
        while time.perf_counter() - t1 < 1.0:
            table.index_select(0, ids_t)
            reps += 1
        tg = (time.perf_counter() - t1) / reps
        gather_cpu = dict(GBps=len(inp) * bytes_per_row / tg / 1e9, ms=tg * 1e3, rows=int(len(inp)),
                          what="torch.index_select on the host table (the reference's CPU gather), "
                               f"{threads} threads")
        del table, ids_t
    model = ""
    try:
        model = next(l.split(":", 1)[1].strip() for l in open("/proc/cpuinfo") if l.startswith("model name"))
    except (OSError, StopIteration):
        pass
    cpu = dict(value=cpu_edges / tc, unit="edges/s", cores=threads, kind="port",
               sample=f"{cpu_batches} batches of the same workload (the timed seed sets, cycled "
                      f"with fresh rng keys) in {tc:.1f} s: sampling, relabel and gather on {threads} "
                      f"OpenMP threads",
               one_thread=one, gather_stage=gather_cpu, host_cpu=model, host_logical_cpus=os.cpu_count())
    del h_indices, h_feats, og, ofs
    return cpu


def main():
    args = parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (no collectives); use --gpus 1")
    if int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: launched with WORLD_SIZE > 1; this build runs on one GPU only")

    import torch

    from apt_amd import capi, synth
    from apt_amd.pipeline import MiniBatchPipeline

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    capi.lib()
    for kv in filter(None, args.tune.split(",")):
        key, val = kv.split("=")
        capi.set_tuning(key, int(val))
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    w = dict(WORKLOADS[args.workload])
    if args.batch_size:
        w["batch"] = args.batch_size
    if args.feature_dtype:
        w["dtype"] = args.feature_dtype
    if args.fan_out:
        w["fan_out"] = [int(x) for x in args.fan_out.split(",")]
    hops = list(reversed(w["fan_out"]))            # reference python/npc/sampler.py:191
    dtype = torch.bfloat16 if w["dtype"] == "bf16" else torch.float32
    esize = 2 if w["dtype"] == "bf16" else 4
    B, K, W = w["batch"], args.steps, args.warmup

    t0 = time.time()
    N = w["nodes"]
    requests = None
    part_note = ""
    P = lo = cache = pos_map = min_vids = None      # only partitioned workloads have them
    if "parts" in w:
        P = w["parts"]
        share = synth.partition_share(N, w["edges"], P, w["part"], w["dim"], dtype, w["cache_ratio"], args.seed, dev)
        lo, hi, indptr, indices, feats = share["lo"], share["hi"], share["indptr"], share["indices"], share["feats"]
        cache, pos_map, min_vids, n_cache = share["cache"], share["pos_map"], share["min_vids"], share["hot"].numel()
        graph = capi.Graph(indptr, indices, row_begin=lo, num_total_nodes=N)
        store = capi.FeatStore(feats, cache, pos_map)
        # bucket 0 is this GPU (reference src/cuda/npc_kernel.cu:398-408), the other owners 1..P-1
        requests = dict(feat_pos_map=pos_map, remote_worker_map=share["remote_worker_map"],
                        min_vids=min_vids, world_size=P, num_remote_workers=P)
        del share
        seed_lo, seed_n = lo, hi - lo
        part_note = (f", rows [{lo}, {hi}) of {P} contiguous parts held here, cache of the {n_cache} "
                     f"hottest remote rows, misses bucketed into {P} owner lists")
    else:
        indptr, indices = synth.rmat_csr_gpu(N, w["edges"], args.seed, dev)
        feats = synth.random_features(N, w["dim"], dtype, args.seed + 1, dev)
        graph = capi.Graph(indptr, indices)
        store = capi.FeatStore(feats)
        seed_lo, seed_n = 0, N
    torch.cuda.synchronize()
    t_setup = time.time() - t0
    num_edges_graph = int(indices.numel())
    max_deg = int((indptr[1:] - indptr[:-1]).max().item())

    def make_pipe(use_graph):
        return MiniBatchPipeline(graph, store, B, hops, replace=args.replace, fused=args.driver != "unfused",
                                 use_graph=use_graph, requests=requests, defer_lookup=args.defer_lookup == "on")

    pipe = make_pipe(args.driver == "graph")
    # the per-stage pass brackets stages with events, which a graph replay does not allow
    stage_pipe = pipe if args.driver != "graph" else make_pipe(False)

    gen = torch.Generator(device=dev)
    gen.manual_seed(args.seed + 2)
    need = (K + W) * B
    if need <= seed_n:
        pool = seed_lo + torch.randperm(seed_n, generator=gen, device=dev)[:need]
        seed_sets = [pool[i * B:(i + 1) * B].contiguous() for i in range(K + W)]
    else:   # more seeds than nodes: each batch still without repetition
        seed_sets = [(seed_lo + torch.randperm(seed_n, generator=gen, device=dev)[:B]).contiguous()
                     for _ in range(K + W)]

    ev = lambda: torch.cuda.Event(enable_timing=True)
    staged = args.driver != "graph"   # a graph replay cannot be bracketed stage by stage

    kev = KernelEvents()           # HIP events that ride on a kernel's dispatch (kernel begin / kernel end)
    H = len(hops)

    def run_step(p, i, gk=None, sk=None):
        seeds, key = seed_sets[i], args.seed + 100 + i
        if gk is None:
            p.run(seeds, key)
            return
        if sk is not None:   # the last hop's sampling kernel records its begin / end
            capi.check(capi.lib().apt_time_next_sample(H - 1, sk[0], sk[1]))
        p.sample(seeds, key, defer_lookup=True)   # as run() does: the relabel's last pass rides in the gather's launch
        capi.check(capi.lib().apt_time_next_gather(gk[0], gk[1]))   # the gather dispatch records its begin / end
        p.gather()

    # ---- warm-up
    for i in range(W):
        run_step(pipe, i)
    torch.cuda.synchronize()

    # ---- timed region: exactly K steps on one stream.  Gather dispatches carry two HIP events that the
    # GPU stamps when the kernel begins and ends (no extra packets on the stream); what is left of the
    # region is sampling + relabel, dispatch gaps included.  Such a dispatch costs the host a little more
    # to enqueue, which would show in launch-bound small workloads, so a limited number of evenly spaced steps (--event_steps) carry them
    # (and the last hop's sampling kernel of the same steps).
    every = max(1, -(-K // max(1, args.event_steps)))
    timed_steps = [i for i in range(K) if staged and i % every == 0]
    gkevs = {i: kev.pair() for i in timed_steps}
    skevs = {i: kev.pair() for i in timed_steps} if args.driver == "fused" else {}
    start, stop = ev(), ev()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    start.record()
    for i in range(K):
        run_step(pipe, W + i, gkevs.get(i), skevs.get(i))
    stop.record()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    sample_us = None
    if staged:
        gather_ms_by_step = [kev.ms(gkevs[i]) for i in timed_steps]
        gather_ms = sorted(gather_ms_by_step)
        t_gather = sum(gather_ms) / len(gather_ms) * K
        t_sample = start.elapsed_time(stop) - t_gather
        if skevs:
            sample_us = {i: kev.ms(skevs[i]) * 1e3 for i in timed_steps}

    # ---- the same K steps once more, one event between steps: the spread of the per-step time
    marks = [ev() for _ in range(K + 1)]
    marks[0].record()
    for i in range(K):
        run_step(pipe, W + i)
        marks[i + 1].record()
    torch.cuda.synchronize()
    per_step_ms = quantiles([marks[i].elapsed_time(marks[i + 1]) for i in range(K)])

    if args.calibration_copy_mib > 0:
        a = torch.ones(args.calibration_copy_mib << 20, dtype=torch.uint8, device=dev)
        b = torch.empty_like(a)
        capi.synth_copy(a, b)
        torch.cuda.synchronize()
        del a, b

    # ---- the same K batches once more, untimed, to read their sizes (one host sync per batch); with the
    # graph driver this pass also provides the stage timings
    edges = rows = 0
    hop_sizes = []
    last_hop = {}        # step -> (frontier rows, sampled edges) of the last hop, for the steps whose kernel was timed
    if not staged:
        t_sample = t_gather = 0.0
    for i in range(K):
        m = (ev(), ev(), ev())
        m[0].record()
        stage_pipe.sample(seed_sets[W + i], args.seed + 100 + W + i, defer_lookup=True)
        m[1].record()
        stage_pipe.gather()
        m[2].record()
        torch.cuda.synchronize()
        if not staged:
            t_sample += m[0].elapsed_time(m[1])
            t_gather += m[1].elapsed_time(m[2])
        sizes = stage_pipe.sizes.cpu().tolist()
        if sample_us is not None and i in sample_us:
            last_hop[i] = (sizes[H - 1], int(stage_pipe.counts[H - 1][:sizes[H - 1]].sum().item()))
        edges += sizes[-1]
        rows += sizes[len(hops)] if requests is None else int(stage_pipe.request_sizes[0].item())
        hop_sizes.append(sizes[:-1])
    request_sizes = None if requests is None else stage_pipe.request_sizes.cpu().tolist()
    # bytes per gathered row: what the launch moves (an identity store has no position map to read) and the
    # figure of the roofline definition (always 16 bytes of id + position)
    bytes_per_row, bytes_per_row_def = gather_bytes_per_row(w["dim"], esize, store.pos_map is not None)
    gather_gbps = rows * bytes_per_row / (t_gather * 1e-3) / 1e9
    edges_per_s = edges / elapsed

    # ---- the same K batches with the relabel's last pass riding in the gather's launch
    # (MiniBatchPipeline(defer_lookup=True)): that launch is then no longer the gather alone, which is why
    # the timed region above, and with it `roofline`, keeps the pass as a launch of its own
    deferred = None
    if args.defer_lookup == "off" and args.driver == "fused" and requests is None:
        dp = MiniBatchPipeline(graph, store, B, hops, replace=args.replace, defer_lookup=True)
        for i in range(W):
            dp.run(seed_sets[i], args.seed + 100 + i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(K):
            dp.run(seed_sets[W + i], args.seed + 100 + W + i)
        torch.cuda.synchronize()
        t_def = time.perf_counter() - t0
        pairs = []
        for i in range(min(K, 25)):
            dp.sample(seed_sets[W + i], args.seed + 100 + W + i, defer_lookup=True)
            pairs.append(kev.pair())
            capi.check(capi.lib().apt_time_next_gather(*pairs[-1]))
            dp.gather()
        torch.cuda.synchronize()
        deferred = {"ms_per_step": t_def / K * 1e3, "edges_per_s": edges / t_def,
                    "gather_launch_with_the_pass_us": sum(kev.ms(pr) for pr in pairs) / len(pairs) * 1e3}
        del dp

    # ---- the same K batches with N batches in flight: N pipelines (own buffers, rank table) on N
    # streams, batches dealt round-robin; reported beside the single-stream figure
    in_flight = None
    if args.inflight > 1:
        pipes, streams = [pipe], [torch.cuda.current_stream()]
        for _ in range(1, args.inflight):
            pipes.append(make_pipe(args.driver == "graph"))
            streams.append(torch.cuda.Stream())
        torch.cuda.synchronize()

        def run_batches(first, count):
            for i in range(count):
                k = i % len(pipes)
                with torch.cuda.stream(streams[k]):
                    pipes[k].run(seed_sets[first + i], args.seed + 100 + first + i)

        run_batches(0, W)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        run_batches(W, K)
        torch.cuda.synchronize()
        t_fl = time.perf_counter() - t0
        assert all(int(p.misses.item()) == 0 for p in pipes)
        in_flight = {"batches_in_flight": len(pipes), "ms_per_step": t_fl / K * 1e3,
                     "edges_per_s": edges / t_fl}
        del pipes[1:]
        # the same through the epoch loader a trainer would use (MiniBatchLoader): the consumer receives
        # every batch narrowed to its sizes, which costs one host read-back per batch
        if args.driver == "fused":
            from apt_amd.loader import MiniBatchLoader
            loader = MiniBatchLoader(graph, store, torch.cat(seed_sets), B, hops, in_flight=args.inflight,
                                     shuffle=False, replace=args.replace, seed=args.seed, requests=requests)
            it = iter(loader)
            for _ in range(W):
                next(it)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            loader_edges = sum(batch["num_edges"] for batch in it)
            torch.cuda.synchronize()
            t_ld = time.perf_counter() - t0
            in_flight["loader"] = {"ms_per_step": t_ld / K * 1e3, "edges_per_s": loader_edges / t_ld}
            del loader, it
    assert int(pipe.misses.item()) == 0 and int(stage_pipe.misses.item()) == 0

    # ---- optional aggregation stage on the outermost block of the last batch
    agg = None
    if args.aggregation:
        agg = stage_aggregation(args=args, capi=capi, dev=dev, K=K, seed_sets=seed_sets,
                                stage_pipe=stage_pipe, synth=synth, torch=torch, W=W)

    # ---- optional: every hop's block as COO + CSC (+ CSR), device-side sizes, after sampling
    fmt = None
    if args.formats:
        fmt = stage_formats(args=args, B=B, ev=ev, graph=graph, hops=hops, K=K,
                            MiniBatchPipeline=MiniBatchPipeline, requests=requests, seed_sets=seed_sets,
                            store=store, torch=torch, W=W)

    # ---- optional: bucketing by owner and pack / unpack of hidden rows (the local halves of feat_shuffle)
    shuffle = None
    if args.shuffle:
        shuffle = stage_shuffle(args=args, capi=capi, dev=dev, hops=hops, N=N, seed_sets=seed_sets,
                                stage_pipe=stage_pipe, torch=torch, W=W)

    # ---- optional: cache construction and the strategy dry run (the callers of the registries)
    cache_build = None
    if args.cache_build and requests is None:
        cache_build = stage_cache_build(args=args, B=B, bytes_per_row=bytes_per_row, capi=capi, dev=dev,
                                        graph=graph, hops=hops, indptr=indptr, N=N, seed_sets=seed_sets,
                                        stage_pipe=stage_pipe, store=store, torch=torch, W=W)

    # ---- CPU baseline: the oracle on this machine's host cores, bounded sample
    cpu = None
    if args.cpu_seconds > 0:
        cpu = stage_cpu_baseline(args=args, bytes_per_row=bytes_per_row, cache=cache, dtype=dtype, feats=feats,
                                 hops=hops, indices=indices, indptr=indptr, K=K, lo=lo, min_vids=min_vids, N=N,
                                 P=P, pos_map=pos_map, requests=requests, seed_sets=seed_sets, torch=torch, W=W)

    # ---- the north-star sentence's own shape: batch 1024 on this graph, bf16 and fp32 rows
    target = None
    if args.target_leg == "on" or (args.target_leg == "auto" and args.workload == "full" and requests is None):
        extra = {}

        def store_of(name):
            want = torch.bfloat16 if name == "bf16" else torch.float32
            if feats.dtype == want:
                return store
            extra.clear()                                  # one extra table at a time
            extra[name] = synth.random_features(N, w["dim"], want, args.seed + 1, dev)
            return capi.FeatStore(extra[name])

        target = stage_target_shape(args=args, capi=capi, dev=dev, graph=graph, hops=hops, kev=kev,
                                    MiniBatchPipeline=MiniBatchPipeline, N=N, seed_n=seed_n, store_of=store_of,
                                    synth=synth, torch=torch)
        extra.clear()
        torch.cuda.empty_cache()

    relabel_small = stage_relabel_small(capi, dev, N, torch) if args.relabel_small else None
    phase_costs = stage_phase_costs(capi, dev, torch) if args.phase_costs else None
    gather_sizes = None
    if args.gather_sizes and requests is None:
        gather_sizes = stage_gather_sizes(capi, dev, kev, store, N, torch)
    frontier_order = None
    if args.frontier_order and requests is None and args.driver == "fused":
        frontier_order = stage_frontier_order(args, capi, dev, graph, hops, seed_sets, stage_pipe, torch, W)

    alternate = None
    if args.alternate and requests is None:
        alternate = stage_alternate(args, capi, graph, hops, kev, MiniBatchPipeline, seed_n, seed_lo, store,
                                    args.alternate_batch or B, torch, dev)

    # ---- what bounds the sampling kernel: random transactions.  The GPU's rate for them, measured here.
    ceilings = stage_ceilings(capi, dev, N, torch) if args.ceilings != "off" else None
    ceilings_by_size = [stage_ceilings(capi, dev, N, torch, int(float(m) * (1 << 20)) // 16 * 16)
                        for m in args.ceiling_table_mib.split(",") if m.strip()] or None
    roofline_sampling = None
    if sample_us and last_hop:
        steps_ = sorted(last_hop)
        us_ = [sample_us[i] for i in steps_]
        r_ = sum(last_hop[i][0] for i in steps_) / len(steps_)
        e_ = sum(last_hop[i][1] for i in steps_) / len(steps_)
        t_ = sum(us_) / len(us_) * 1e-6
        alg = 24 * r_ + 16 * e_ + (8 * r_ if graph.adj_pos_map is not None else 0)
        # per frontier row one random line for its indptr pair, per sampled slot one random index load and one
        # random rank-table read (atomics for the slots that bid come on top and are not counted here)
        acc = r_ + 2 * e_
        q = quantiles(us_)
        # new nodes of the hop: each costs at least one atomic (the bid that ends up owning it)
        new_nodes = sum(hop_sizes[i][H] - hop_sizes[i][H - 1] for i in steps_) / len(steps_)
        bound_us = None
        if ceilings:
            bound_us = (acc / ceilings["load_G_per_s"] + new_nodes / ceilings["atomic_min_returning_G_per_s"]) * 1e-3
        roofline_sampling = {
            "bound": "hbm", "kernel": f"sample_kernel, hop {H} of {H} (fanout {hops[-1]}), rank-table bids included",
            "achieved": alg / t_ / 1e9, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": alg / t_ / 1e9 / HBM_PEAK_GBPS,
            "traffic": None, "algorithmic_bytes_per_launch": alg, "bytes_per_row": "24 + 16 k, k = min(fanout, degree)",
            "rows_per_launch": r_, "edges_per_launch": e_, "avg_launch_us": t_ * 1e6,
            "launch_us_min_median_max": [q["min"], q["median"], q["max"]],
            "random_accesses_per_launch": acc, "random_accesses_G_per_s": acc / t_ / 1e9,
            "random_load_ceiling_G_per_s": ceilings["load_G_per_s"] if ceilings else None,
            "frac_of_random_load_ceiling": acc / t_ / 1e9 / ceilings["load_G_per_s"] if ceilings else None,
            # the time those loads and one atomic per new node take at this GPU's measured rates for them
            "new_nodes_per_launch": new_nodes,
            "random_atomic_ceiling_G_per_s": ceilings["atomic_min_returning_G_per_s"] if ceilings else None,
            "transaction_bound_us": bound_us, "frac_of_transaction_bound": bound_us / (t_ * 1e6) if bound_us else None,
            "timing": f"HIP events carried by {len(steps_)} of the {K} dispatches of the timed region",
        }

    tkey = (args.workload, w["dtype"], w["dim"], B)
    traffic_row = MEASURED_GATHER_TRAFFIC_PER_ROW.get(tkey) if not args.fan_out and requests is None else None

    out = {
        "metric": "sampled edges/s (3-hop 15,10,5) + feature-gather GB/s as % of HBM peak",
        "value": edges_per_s,
        "unit": "edges/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": W,
        "ms_per_step": elapsed / K * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int64",
        "data": "synthetic",
        "config": {
            "workload": f"{args.workload}: R-MAT {w['nodes']} nodes / {num_edges_graph} directed edges "
                        f"(max degree {max_deg}), features {w['dim']} x {w['dtype']}, batch {B}, "
                        f"fan_out {w['fan_out']} (hops from the seeds: {hops}), "
                        f"{'with' if args.replace else 'without'} replacement, relabel per hop, "
                        f"gather of all input nodes" + part_note,
            "batch": B, "fan_out": w["fan_out"], "feature_dtype": w["dtype"], "driver": args.driver,
            "graph": "R-MAT a=.57 b=.19 c=.19, CSR built on the GPU: multigraph rows (an id may repeat in a row), "
                     "unsorted, no dedup",
        },
        "roofline": {
            "bound": "hbm", "kernel": "gather_kernel",
            "achieved": gather_gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": gather_gbps / HBM_PEAK_GBPS,
            "traffic": traffic_row[0] * rows / K if traffic_row else None,
            "traffic_source": traffic_row[1] if traffic_row else None,
            "algorithmic_bytes_per_launch": bytes_per_row * rows / K,
            "bytes_per_row": bytes_per_row, "rows_per_launch": rows / K,
            # the roofline definition charges 16 bytes of id + position per row whether or not the store has a
            # position map; achieved / frac above use the bytes this launch moves
            "bytes_per_row_definition": bytes_per_row_def,
            "frac_by_definition_bytes": gather_gbps / HBM_PEAK_GBPS * bytes_per_row_def / bytes_per_row,
            "avg_launch_us": t_gather / K * 1e3,
            "launch_us_min_median_max": ([gather_ms[0] * 1e3, gather_ms[len(gather_ms) // 2] * 1e3,
                                          gather_ms[-1] * 1e3] if staged else None),
            "launch_us_by_timed_step": ({str(i): round(t * 1e3, 2) for i, t in zip(timed_steps, gather_ms_by_step)}
                                        if staged else None),
            "timing": (f"HIP events carried by {len(timed_steps)} of the {K} gather dispatches of the timed region "
                       f"(kernel begin / end)" if staged else "HIP events recorded around each gather launch of an untimed pass"),
            # with the pipeline's default the batch's last relabel pass rides in the first workgroups of this launch
            # (--defer_lookup off launches it on its own before the gather); its bytes are not counted above
            "launch_also_carries": ("the batch's last relabel pass (rank-table lookups of the slots that lost a race)"
                                    if pipe.can_defer_lookup else None),
        },
        "roofline_sampling": roofline_sampling,
        "cpu_baseline": cpu,
        "aggregation": agg,
        "block_formats": fmt,
        "cache_build": cache_build,
        "shuffle": shuffle,
        "relabel_small": relabel_small,
        "phase_costs": phase_costs,
        "alternate": alternate,
        "gather_sizes": gather_sizes,
        "frontier_order": frontier_order,
        "stages": {
            "target_shape": target,
            "per_step_ms": per_step_ms,
            "random_access_ceilings": ceilings,
            "random_access_by_table_size": ceilings_by_size,
            "in_flight": in_flight,
            "deferred_lookup": deferred,
            "edges_per_step": edges / K,
            "input_nodes_per_step": rows / K,
            "sample_relabel_ms": t_sample / K,
            "gather_ms": t_gather / K,
            "sample_relabel_edges_per_s": edges / (t_sample * 1e-3),
            "frontier_sizes_last_step": hop_sizes[-1],
            "request_bucket_sizes_last_step": request_sizes,
            "setup_s": t_setup,
        },
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
