#!/usr/bin/env python3
"""Mini-batch construction benchmark on one MI355X.

A step is one mini-batch: multi-hop uniform neighbour sampling without
replacement + relabel on every hop + feature gather of the input nodes, with
the graph, the feature table and the seeds resident in HBM.  K steps are timed
back to back on one stream.  Prints ONE JSON line: sampled edges/s for the
whole step, the gather kernel's achieved HBM bandwidth against the 8 TB/s peak
(roofline, from HIP events carried by gather dispatches of the timed region),
and the CPU oracle timed on this machine's host cores on a bounded sample of
the same workload (cpu_baseline), whose first batch is also compared bit for bit
with the GPU's (cpu_baseline.parity; a mismatch ends the run with an error).
stages.in_flight is the same K batches with several batches in flight on
separate streams; stages.configs repeats the measurement on the other
configurations (medium, one partition's share, the small plumbing case) and
times the aggregation kernels on the partition's outermost block.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload full|target|medium|partition|small]
"""
import argparse
import ctypes
import json
import os
import sys
import time
from types import SimpleNamespace

from bench_extra import HBM_PEAK_GBPS, gather_bytes_per_row, quantiles

# HBM bytes the gather kernel moves per gathered row, from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE runs of
# this script, each scaled by what the same counter reads for the plain copy kernel.  Keyed by everything the
# figure depends on, (workload, graph kind, feature dtype, feature dim, batch); a run with any other combination
# reports traffic null.  Each entry names the profiles/ file that holds the counter readings.
MEASURED_GATHER_TRAFFIC_PER_ROW = {
    ("full", "symmetric", "bf16", 128, 4096): (520.4, "profiles/gather_kernel_full_pmc.txt"),
    ("target", "symmetric", "bf16", 128, 1024): (519.5, "profiles/gather_kernel_target_bf16_pmc.txt"),
    ("target", "symmetric", "fp32", 128, 1024): (1030.7, "profiles/gather_kernel_target_fp32_pmc.txt"),
    ("medium", "symmetric", "fp32", 100, 1024): (916.6, "profiles/gather_kernel_medium_pmc.txt"),
    ("partition", "symmetric", "fp32", 128, 1024): (1197.7, "profiles/gather_kernel_partition_pmc.txt"),
    ("small", "directed", "fp32", 128, 1024): (1054.7, "profiles/gather_kernel_small_pmc.txt"),
}
# The same for the last hop's sampling kernel (rank-table bids included): HBM bytes per sampled edge.
MEASURED_SAMPLE_TRAFFIC_PER_EDGE = {
    ("full", "symmetric", "bf16", 128, 4096): (257.7, "profiles/gather_kernel_full_pmc.txt"),
    ("target", "symmetric", "bf16", 128, 1024): (259.8, "profiles/gather_kernel_target_bf16_pmc.txt"),
    ("target", "symmetric", "fp32", 128, 1024): (259.7, "profiles/gather_kernel_target_fp32_pmc.txt"),
    ("medium", "symmetric", "fp32", 100, 1024): (220.1, "profiles/gather_kernel_medium_pmc.txt"),
    ("partition", "symmetric", "fp32", 128, 1024): (417.5, "profiles/gather_kernel_partition_pmc.txt"),
    ("small", "directed", "fp32", 128, 1024): (201.9, "profiles/gather_kernel_small_pmc.txt"),
}

WORKLOADS = {
    # full-scale single GPU: 111M nodes, 1.6B edges stored in both directions, 128 x bf16, batch 4096
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
    # the small plumbing case: 100k nodes, directed, 2 hops
    "small": dict(nodes=100_000, edges=1_500_000, dim=128, dtype="fp32", batch=1024, fan_out=[10, 5]),
}


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="full", choices=sorted(WORKLOADS))
    ap.add_argument("--graph", default="symmetric", choices=["symmetric", "independent"],
                    help="symmetric: every R-MAT edge stored in both directions, a self-loop per node, rows sorted, "
                         "repeated entries merged (the kind of graph the reference trains on); independent: the "
                         "directed edges drawn independently, unsorted multigraph rows.  The small workload is "
                         "always its own directed, deduplicated graph built on the host")
    ap.add_argument("--batch_size", type=int, default=None)
    ap.add_argument("--feature_dtype", default=None, choices=["fp32", "bf16"])
    ap.add_argument("--fan_out", type=str, default=None,
                    help="comma list, k-hop..1-hop as in the reference (the seeds use the last entry)")
    ap.add_argument("--replace", action="store_true", help="sample with replacement (reference semantics)")
    ap.add_argument("--cpu_seconds", type=float, default=12.0,
                    help="seconds of CPU-oracle work for the cpu_baseline leg (0 = skip, also skips its parity check)")
    ap.add_argument("--cpu_threads", type=int, default=None)
    ap.add_argument("--seed", type=int, default=1)
    ap.add_argument("--driver", default="fused", choices=["graph", "fused", "unfused", "unfused_pass", "unfused_hash"],
                    help="graph: fused C driver replayed as a HIP graph; fused: same, launched eagerly; "
                         "unfused: the reference's call pattern, a sampling call and a relabel call per hop, the "
                         "relabel through the graph's rank table with its bids placed by the sampling call "
                         "(apt_sample_neighbors_bidding + apt_relabel_ranked); unfused_pass: the same with the bids "
                         "as a pass of the relabel call; unfused_hash: with the hash-table relabel (apt_relabel)")
    ap.add_argument("--inflight", type=int, default=4,
                    help="after the timed single-stream region, also run the K batches with N of them in "
                         "flight (N pipelines on N HIP streams) and report it under stages.in_flight; 1 = skip")
    ap.add_argument("--configs", default="auto", choices=["auto", "on", "off"],
                    help="after the main workload also measure medium, partition and small and the aggregation "
                         "kernels on the partition's block (stages.configs); auto = only for workload full")
    ap.add_argument("--config_steps", type=int, default=50)
    ap.add_argument("--calibration_copy_mib", type=int, default=0,
                    help="also launch the plain copy kernel once on this many MiB (for scaling "
                         "FETCH_SIZE / WRITE_SIZE when the run is under rocprofv3 --pmc)")
    ap.add_argument("--formats", action="store_true",
                    help="also time the emission of every hop's block as COO + CSC (+ CSR)")
    ap.add_argument("--aggregation", action="store_true",
                    help="also time GraphSAGE-style SpMM (hidden 256, fp32 and bf16) and SDDMM on the "
                         "outermost sampled block of the last batch of this workload")
    ap.add_argument("--shuffle", action="store_true",
                    help="also time the local halves of the feature shuffle on the batch's input nodes: bucketing by "
                         "owner (cluster_permute) and pack / unpack of hidden rows")
    ap.add_argument("--cache_build", action="store_true",
                    help="also time the cache-construction kernels (access counting, cached CSR of the hottest rows, "
                         "cached feature table) and one step of the all-strategies dry run")
    ap.add_argument("--operators", action="store_true",
                    help="also time the batch through the operator layer (per-hop calls and sample_blocks)")
    ap.add_argument("--gather_sizes", action="store_true",
                    help="also time the gather kernel alone on 0 .. 940 k random rows of this workload's table "
                         "(device-side count, every launch with its own events): what a launch costs before it moves a byte")
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
    return ap.parse_args()


class KernelEvents:
    """Pairs of HIP events that ride on a kernel dispatch (kernel begin / kernel end), see
    apt_time_next_gather / apt_time_next_sample."""

    def __init__(self):
        self.hip = ctypes.CDLL("libamdhip64.so")
        self.hip.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        self.hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
        self.hip.hipEventDestroy.argtypes = [ctypes.c_void_p]
        self.hip.hipEventRecord.argtypes = [ctypes.c_void_p, ctypes.c_void_p]

    def pair(self):
        a, b = ctypes.c_void_p(), ctypes.c_void_p()
        assert self.hip.hipEventCreate(ctypes.byref(a)) == 0 and self.hip.hipEventCreate(ctypes.byref(b)) == 0
        return a, b

    def record(self, event, stream):
        """Records `event` on a torch stream."""
        rc = self.hip.hipEventRecord(event, ctypes.c_void_p(stream.cuda_stream))
        assert rc == 0, f"hipEventRecord -> {rc}"

    def destroy(self, pair):
        self.hip.hipEventDestroy(pair[0])
        self.hip.hipEventDestroy(pair[1])

    def ms(self, pair, destroy=True):
        ms = ctypes.c_float()
        rc = self.hip.hipEventElapsedTime(ctypes.byref(ms), pair[0], pair[1])
        assert rc == 0, f"hipEventElapsedTime -> {rc}"
        if destroy:
            self.hip.hipEventDestroy(pair[0])
            self.hip.hipEventDestroy(pair[1])
        return ms.value


# ------------------------------------------------------------------------------------------------ workloads
def build_workload(args, name, w, ctx, full_graph=None):
    """The graph, the feature store and (partitioned workloads) the request description of workload `name`,
    resident in HBM.  full_graph: (indptr, indices) of the 111 M-node graph when the caller already holds it
    (the partition workload is a slice of its rows).  -> SimpleNamespace"""
    torch, capi, synth, dev = ctx.torch, ctx.capi, ctx.synth, ctx.dev
    t0 = time.time()
    N = w["nodes"]
    dtype = torch.bfloat16 if w["dtype"] == "bf16" else torch.float32
    wl = SimpleNamespace(name=name, w=w, N=N, dtype=dtype, esize=2 if w["dtype"] == "bf16" else 4, requests=None,
                         part_note="", P=None, lo=None, cache=None, pos_map=None, min_vids=None, gen_stats={})
    symmetric = args.graph == "symmetric"
    if "parts" in w:
        P = w["parts"]
        if symmetric and full_graph is None:
            full_graph = synth.rmat_symmetric_csr_gpu(N, w["edges"], args.seed, dev, stats=wl.gen_stats)
        share = synth.partition_share(N, w["edges"], P, w["part"], w["dim"], dtype, w["cache_ratio"], args.seed, dev,
                                      full_graph=full_graph if symmetric else None)
        del full_graph
        lo, hi = share["lo"], share["hi"]
        wl.indptr, wl.indices, wl.feats = share["indptr"], share["indices"], share["feats"]
        wl.cache, wl.pos_map, wl.min_vids = share["cache"], share["pos_map"], share["min_vids"]
        wl.graph = capi.Graph(wl.indptr, wl.indices, row_begin=lo, num_total_nodes=N)
        wl.store = capi.FeatStore(wl.feats, wl.cache, wl.pos_map)
        # bucket 0 is this GPU (reference src/cuda/npc_kernel.cu:398-408), the other owners 1..P-1
        wl.requests = dict(feat_pos_map=wl.pos_map, remote_worker_map=share["remote_worker_map"],
                           min_vids=wl.min_vids, world_size=P, num_remote_workers=P)
        wl.P, wl.lo, wl.seed_lo, wl.seed_n = P, lo, lo, hi - lo
        wl.part_note = (f", rows [{lo}, {hi}) of {P} contiguous parts held here, cache of the "
                        f"{share['hot'].numel()} remote rows of largest degree, misses bucketed into {P} owner lists")
        del share
    else:
        if name == "small":
            ip, ix = synth.rmat_csr_numpy(N, w["edges"], args.seed)
            wl.indptr, wl.indices = torch.from_numpy(ip).to(dev), torch.from_numpy(ix).to(dev)
        elif full_graph is not None:
            wl.indptr, wl.indices = full_graph
        elif symmetric:
            wl.indptr, wl.indices = synth.rmat_symmetric_csr_gpu(N, w["edges"], args.seed, dev, stats=wl.gen_stats)
        else:
            wl.indptr, wl.indices = synth.rmat_csr_gpu(N, w["edges"], args.seed, dev)
        wl.feats = synth.random_features(N, w["dim"], dtype, args.seed + 1, dev)
        wl.graph = capi.Graph(wl.indptr, wl.indices)
        wl.store = capi.FeatStore(wl.feats)
        wl.seed_lo, wl.seed_n = 0, N
    torch.cuda.synchronize()
    wl.setup_s = time.time() - t0
    wl.num_edges_graph = int(wl.indices.numel())
    wl.max_deg = int((wl.indptr[1:] - wl.indptr[:-1]).max().item())
    if name == "small":
        wl.graph_kind, wl.graph_note = "directed", ("R-MAT a=.57 b=.19 c=.19 built on the host: directed, repeated "
                                                    "edges removed, rows sorted")
    elif symmetric:
        wl.graph_kind = "symmetric"
        merged = wl.gen_stats.get("merged_fraction")
        wl.graph_note = ("R-MAT a=.57 b=.19 c=.19, symmetrised, self-loops, simple: every drawn edge stored in both "
                         "directions, a self-loop on every node, rows sorted, repeated entries merged"
                         + (f" ({100 * merged:.1f} % of {wl.gen_stats['entries_before_merge']} entries were repeats)"
                            if merged is not None else ""))
    else:
        wl.graph_kind = "independent"
        wl.graph_note = ("R-MAT a=.57 b=.19 c=.19, CSR built on the GPU: directed edges drawn independently, "
                         "multigraph rows (an id may repeat in a row), unsorted, no self-loops")
    return wl


class TraceMarkers:
    """Phase boundaries that show in a kernel trace: a one-workgroup launch of the plain copy kernel between the
    benchmark's phases (the GPU idle before and after it), named in launch order in stages.trace_markers, so that
    a rocprofv3 trace of this command can be cut into the phases the figures of the line come from."""

    def __init__(self, torch, capi, dev):
        self.torch, self.capi = torch, capi
        self.a = torch.zeros(16, dtype=torch.uint8, device=dev)
        self.b = torch.zeros(16, dtype=torch.uint8, device=dev)
        self.names = []

    def __call__(self, name):
        self.torch.cuda.synchronize()
        self.capi.synth_copy(self.a, self.b)
        self.torch.cuda.synchronize()
        self.names.append(name)


def driver_kw(args):
    """MiniBatchPipeline arguments of --driver."""
    if args.driver in ("fused", "graph"):
        return dict(fused=True)
    return dict(fused=False, relabel={"unfused": "ranked_bidding", "unfused_pass": "ranked"}.get(args.driver, "hash"))


def make_seed_sets(ctx, wl, B, count, seed):
    torch, dev = ctx.torch, ctx.dev
    gen = torch.Generator(device=dev)
    gen.manual_seed(seed)
    need = count * B
    if need <= wl.seed_n:
        pool = wl.seed_lo + torch.randperm(wl.seed_n, generator=gen, device=dev)[:need]
        return [pool[i * B:(i + 1) * B].contiguous() for i in range(count)]
    # more seeds than nodes: each batch still without repetition
    return [(wl.seed_lo + torch.randperm(wl.seed_n, generator=gen, device=dev)[:B]).contiguous() for _ in range(count)]


# ------------------------------------------------------------------------------------------------ measurement
def measure(args, ctx, wl, B, hops, K, W, event_steps, per_step=True, tag=""):
    """W warm-up and exactly K timed batches of workload wl on one stream, then (untimed) the same batches
    again to read their sizes.  -> SimpleNamespace with the pipeline, the seed sets and the figures."""
    torch, capi, kev = ctx.torch, ctx.capi, ctx.kev
    from apt_amd.pipeline import MiniBatchPipeline

    def make_pipe(use_graph):
        return MiniBatchPipeline(wl.graph, wl.store, B, hops, replace=args.replace, use_graph=use_graph,
                                 requests=wl.requests, defer_lookup=args.defer_lookup == "on", **driver_kw(args))

    m = SimpleNamespace(make_pipe=make_pipe, B=B, hops=hops, K=K, W=W)
    pipe = m.pipe = make_pipe(args.driver == "graph")
    # the per-stage pass brackets stages with events, which a graph replay does not allow
    stage_pipe = m.stage_pipe = pipe if args.driver != "graph" else make_pipe(False)
    seed_sets = m.seed_sets = make_seed_sets(ctx, wl, B, K + W, args.seed + 2)
    staged = m.staged = args.driver != "graph"
    H = len(hops)
    ev = lambda: torch.cuda.Event(enable_timing=True)

    def run_step(p, i, gk=None, sk=None):
        seeds, key = seed_sets[i], args.seed + 100 + i
        if gk is None:
            p.run(seeds, key)
            return
        if sk is not None:   # the last hop's sampling kernel records its begin / end
            capi.check(capi.lib().apt_time_next_sample(H - 1, sk[0], sk[1]))
        p.sample(seeds, key, defer_lookup=True)   # as run() does
        capi.check(capi.lib().apt_time_next_gather(gk[0], gk[1]))   # the gather dispatch records its begin / end
        p.gather()

    m.run_step = run_step
    for i in range(W):
        run_step(pipe, i)
    torch.cuda.synchronize()

    # ---- timed region: exactly K steps on one stream.  Gather dispatches carry two HIP events that the
    # GPU stamps when the kernel begins and ends (no extra packets on the stream); what is left of the
    # region is sampling + relabel, dispatch gaps included.  Such a dispatch costs the host a little more
    # to enqueue, which would show in launch-bound small workloads, so a limited number of evenly spaced
    # steps (--event_steps) carry them (and the last hop's sampling kernel of the same steps), and never more
    # than every fourth: a dispatch with events is fenced off from its neighbours on the stream, about 4 us
    # each, which a short region (--steps 20) would otherwise pay on every step.
    every = max(min(4, K), -(-K // max(1, event_steps)))
    timed_steps = m.timed_steps = [i for i in range(K) if staged and i % every == 0]
    gkevs = {i: kev.pair() for i in timed_steps}
    skevs = {i: kev.pair() for i in timed_steps} if args.driver == "fused" else {}
    start, stop = ev(), ev()
    ctx.mark(f"{tag}timed region: {K} batches on one stream")
    t0 = time.perf_counter()
    start.record()
    for i in range(K):
        run_step(pipe, W + i, gkevs.get(i), skevs.get(i))
    stop.record()
    torch.cuda.synchronize()
    m.elapsed = time.perf_counter() - t0
    ctx.mark(f"{tag}end of the timed region")
    m.sample_us = None
    if staged:
        m.gather_ms_by_step = [kev.ms(gkevs[i]) for i in timed_steps]
        m.gather_ms = sorted(m.gather_ms_by_step)
        m.t_gather = sum(m.gather_ms) / len(m.gather_ms) * K
        m.t_sample = start.elapsed_time(stop) - m.t_gather
        if skevs:
            m.sample_us = {i: kev.ms(skevs[i]) * 1e3 for i in timed_steps}

    # ---- the same K steps once more, one event between steps: the spread of the per-step time
    m.per_step_ms = None
    if per_step:
        marks = [ev() for _ in range(K + 1)]
        marks[0].record()
        for i in range(K):
            run_step(pipe, W + i)
            marks[i + 1].record()
        torch.cuda.synchronize()
        m.per_step_ms = quantiles([marks[i].elapsed_time(marks[i + 1]) for i in range(K)])

    # ---- the same K batches once more, untimed, to read their sizes (one host sync per batch); with the
    # graph driver this pass also provides the stage timings
    m.edges = m.rows = 0
    m.hop_sizes = []
    m.last_hop = {}     # step -> (frontier rows, sampled edges) of the last hop, for the steps whose kernel was timed
    if not staged:
        m.t_sample = m.t_gather = 0.0
    for i in range(K):
        mk = (ev(), ev(), ev())
        mk[0].record()
        stage_pipe.sample(seed_sets[W + i], args.seed + 100 + W + i, defer_lookup=True)
        mk[1].record()
        stage_pipe.gather()
        mk[2].record()
        torch.cuda.synchronize()
        if not staged:
            m.t_sample += mk[0].elapsed_time(mk[1])
            m.t_gather += mk[1].elapsed_time(mk[2])
        sizes = stage_pipe.sizes.cpu().tolist()
        if m.sample_us is not None and i in m.sample_us:
            m.last_hop[i] = (sizes[H - 1], int(stage_pipe.counts[H - 1][:sizes[H - 1]].sum().item()))
        m.edges += sizes[-1]
        m.rows += sizes[H] if wl.requests is None else int(stage_pipe.request_sizes[0].item())
        m.hop_sizes.append(sizes[:-1])
    m.request_sizes = None if wl.requests is None else stage_pipe.request_sizes.cpu().tolist()
    # bytes per gathered row: what the launch moves (an identity store has no position map to read) and the
    # figure of the roofline definition (always 16 bytes of id + position)
    m.bytes_per_row, m.bytes_per_row_def = gather_bytes_per_row(wl.w["dim"], wl.esize, wl.store.pos_map is not None)
    m.gather_gbps = m.rows * m.bytes_per_row / (m.t_gather * 1e-3) / 1e9
    m.edges_per_s = m.edges / m.elapsed
    assert int(pipe.misses.item()) == 0 and int(stage_pipe.misses.item()) == 0
    return m


def traffic_entry(table, args, wl, B):
    if args.fan_out or args.replace or args.tune:
        return None           # counters were read with the shipped kernels on the workload's own shape
    return table.get((wl.name, wl.graph_kind, wl.w["dtype"], wl.w["dim"], B))


def gather_roofline(args, wl, m, pipe_defers):
    K = m.K
    tr = traffic_entry(MEASURED_GATHER_TRAFFIC_PER_ROW, args, wl, m.B)
    return {
        "bound": "hbm", "kernel": "gather_kernel",
        "achieved": m.gather_gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
        "frac": m.gather_gbps / HBM_PEAK_GBPS,
        "traffic": tr[0] * m.rows / K if tr else None,
        "traffic_source": tr[1] if tr else None,
        "algorithmic_bytes_per_launch": m.bytes_per_row * m.rows / K,
        "bytes_per_row": m.bytes_per_row, "rows_per_launch": m.rows / K,
        # the roofline definition charges 16 bytes of id + position per row whether or not the store has a
        # position map; achieved / frac above use the bytes this launch moves
        "bytes_per_row_definition": m.bytes_per_row_def,
        "frac_by_definition_bytes": m.gather_gbps / HBM_PEAK_GBPS * m.bytes_per_row_def / m.bytes_per_row,
        "avg_launch_us": m.t_gather / K * 1e3,
        "launch_us_min_median_max": ([m.gather_ms[0] * 1e3, m.gather_ms[len(m.gather_ms) // 2] * 1e3,
                                      m.gather_ms[-1] * 1e3] if m.staged else None),
        "launch_us_by_timed_step": ({str(i): round(t * 1e3, 2) for i, t in zip(m.timed_steps, m.gather_ms_by_step)}
                                    if m.staged else None),
        "timing": (f"HIP events carried by {len(m.timed_steps)} of the {K} gather dispatches of the timed region "
                   f"(kernel begin / end)" if m.staged else "HIP events recorded around each gather launch of an untimed pass"),
        # with defer_lookup on, the batch's last relabel pass rides in the first workgroups of this launch
        "launch_also_carries": ("the batch's last relabel pass (rank-table lookups of the slots that lost a race)"
                                if pipe_defers else None),
    }


def sampling_roofline(args, wl, m, ceilings):
    if not (m.sample_us and m.last_hop):
        return None
    H, hops, K = len(m.hops), m.hops, m.K
    steps_ = sorted(m.last_hop)
    us_ = [m.sample_us[i] for i in steps_]
    r_ = sum(m.last_hop[i][0] for i in steps_) / len(steps_)
    e_ = sum(m.last_hop[i][1] for i in steps_) / len(steps_)
    t_ = sum(us_) / len(us_) * 1e-6
    alg = 24 * r_ + 16 * e_ + (8 * r_ if wl.graph.adj_pos_map is not None else 0)
    # per frontier row one random line for its indptr pair, per sampled slot one random index load and one
    # random rank-table read (atomics for the slots that bid come on top and are not counted here)
    acc = r_ + 2 * e_
    q = quantiles(us_)
    # new nodes of the hop: each costs at least one atomic (the bid that ends up owning it)
    new_nodes = sum(m.hop_sizes[i][H] - m.hop_sizes[i][H - 1] for i in steps_) / len(steps_)
    bound_us = None
    if ceilings:
        bound_us = (acc / ceilings["load_G_per_s"] + new_nodes / ceilings["atomic_min_returning_G_per_s"]) * 1e-3
    tr = traffic_entry(MEASURED_SAMPLE_TRAFFIC_PER_EDGE, args, wl, m.B)
    return {
        "bound": "hbm", "kernel": f"sample_kernel, hop {H} of {H} (fanout {hops[-1]}), rank-table bids included",
        "achieved": alg / t_ / 1e9, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": alg / t_ / 1e9 / HBM_PEAK_GBPS,
        "traffic": tr[0] * e_ if tr else None, "traffic_source": tr[1] if tr else None,
        "algorithmic_bytes_per_launch": alg, "bytes_per_row": "24 + 16 k, k = min(fanout, degree)",
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


def stage_target_shape(args, ctx, wl, hops, store_of):
    """Batch 1024 on the same graph with 128 x bf16 and 128 x fp32 rows: the shape the gather target
    (>= 60 % of HBM peak) is stated on.  Every gather dispatch carries events; the sizes of every batch are
    kept on the device and read afterwards, so each launch's rows and duration give its own fraction.
    The figures are of the gather kernel launched by itself (the relabel's last pass as a launch of its own
    before it); the pipeline's default lets that pass ride in the gather's launch, which makes the batch
    shorter and that launch a little longer: `with_lookup_riding` has the same batches that way.  `loader` is
    the epoch loader's rate on the same batches (several in flight, sizes read back by the host)."""
    torch, capi, kev, dev = ctx.torch, ctx.capi, ctx.kev, ctx.dev
    from apt_amd.loader import MiniBatchLoader
    from apt_amd.pipeline import MiniBatchPipeline
    B, Kt, Wt, H = 1024, args.target_steps, 20, len(hops)
    gen = torch.Generator(device=dev)
    gen.manual_seed(args.seed + 77)
    out = {"batch": B, "batches": Kt, "warmup": Wt}
    for name in ("bf16", "fp32"):
        store = store_of(name)
        esize = store.local_table.element_size()
        moved, spec = gather_bytes_per_row(store.out_dim, esize, store.pos_map is not None)
        pipe = MiniBatchPipeline(wl.graph, store, B, hops, replace=args.replace, defer_lookup=args.defer_lookup == "on",
                                 **driver_kw(args))
        pool = torch.randperm(wl.seed_n, generator=gen, device=dev)[:(Kt + Wt) * B]
        sets = [pool[i * B:(i + 1) * B].contiguous() for i in range(Kt + Wt)]
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

        ctx.mark(f"target shape {name}: {Kt} batches of 1024, every gather dispatch with events")
        us, rows, frac, step_ms = timed_pass(False)
        ctx.mark(f"end of target shape {name}")
        edges = log[:, H + 1].cpu().tolist()
        wall_alone = wall_pass(False)
        riding = None
        if pipe.can_defer_lookup:
            us_r, _, frac_r, _ = timed_pass(True)
            riding = {"us_median": quantiles(us_r)["median"], "frac": quantiles(frac_r)["median"],
                      "frac_p10": quantiles(frac_r)["p10"], "ms_per_step": wall_pass(True) * 1e3}
        wall = riding["ms_per_step"] * 1e-3 if riding else wall_alone     # what a pipeline does by default
        del pipe
        loader_fig = None
        if args.driver == "fused" and args.inflight > 1:
            loader = MiniBatchLoader(wl.graph, store, torch.cat(sets), B, hops, in_flight=args.inflight,
                                     shuffle=False, replace=args.replace, seed=args.seed)
            t_ld, l_edges, gaps = time_loader(torch, loader, Wt)
            loader_fig = {"batches_in_flight": args.inflight, "ms_per_step": t_ld / Kt * 1e3,
                          "edges_per_s": l_edges / t_ld, "ms_between_batches": gaps,
                          "host_us_per_batch": loader_cost_per_batch(loader)}
            del loader
        q_us, q_frac = quantiles(us), quantiles(frac)
        tr = MEASURED_GATHER_TRAFFIC_PER_ROW.get(("target", wl.graph_kind, name, store.out_dim, B), (None, None))
        out[name] = {
            "rows": sum(rows) / Kt, "bytes_per_row": moved, "bytes_per_row_definition": spec,
            "us_median": q_us["median"], "us_p10": q_us["p10"], "us_p90": q_us["p90"], "us_min": q_us["min"],
            "us_max": q_us["max"],
            # fraction of 8 TB/s of each launch (its own rows over its own duration); p10 = the slow end
            "frac": q_frac["median"], "frac_p10": q_frac["p10"], "frac_p90": q_frac["p90"],
            "frac_min": q_frac["min"], "frac_max": q_frac["max"],
            "frac_by_definition_bytes": q_frac["median"] * spec / moved,
            "traffic_bytes_per_row": tr[0], "traffic_source": tr[1],
            "GBps_median": q_frac["median"] * HBM_PEAK_GBPS,
            "ms_per_step": wall * 1e3, "ms_per_step_gather_launched_alone": wall_alone * 1e3,
            "ms_per_step_events": quantiles(step_ms),
            "edges_per_s": sum(edges) / Kt / wall,
            "with_lookup_riding": riding,
            "loader": loader_fig,
        }
        del log, sets, pool
    return out


def quiet_gc():
    """Python's cycle collector walks every container object of the process when it runs a full collection
    (tens of milliseconds with torch imported), and the loops below allocate enough small objects per batch to
    set one off inside a timed region now and then.  Everything alive after set-up is moved out of its reach;
    the garbage of the timed loops themselves is still collected."""
    import gc
    gc.collect()
    gc.freeze()


def time_loader(torch, loader, warm):
    """One epoch of `loader`; the clock starts when the `warm`-th batch has been handed over and stops when the
    last one has (a batch is complete on the GPU when the loader yields it) -> (seconds, sampled edges of the
    timed batches, quantiles of the time between consecutive batches in ms).  The pipeline is not drained before
    the clock starts: the batches the driver has enqueued ahead by then are the steady state, and draining them
    first would hand the timed part that many finished batches for nothing."""
    it = iter(loader)
    stamps = [time.perf_counter()]
    for _ in range(warm):
        next(it)
        stamps[0] = time.perf_counter()
    edges = 0
    for batch in it:
        edges += batch["num_edges"]
        stamps.append(time.perf_counter())
    torch.cuda.synchronize()
    return stamps[-1] - stamps[0], edges, quantiles([(b - a) * 1e3 for a, b in zip(stamps, stamps[1:])])


def loader_cost_per_batch(loader):
    """What a batch costs the host through the loader's C driver, in us: the driver thread's enqueue calls, and
    the consumer's waits for that thread and for the GPU."""
    c = loader.host_cost()
    if not c or not c["batches"]:
        return None
    return {k.replace("_seconds", ""): v / c["batches"] * 1e6 for k, v in c.items() if k != "batches"}


def stage_ceilings(ctx, N):
    """The GPU's rate for one random 4-byte access per work item into a table of the rank table's size."""
    torch, capi, dev = ctx.torch, ctx.capi, ctx.dev
    nbytes = max(1 << 20, (N * 4 + 15) // 16 * 16)
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
            capi.synth_random_access(mode, table, n, rep + 1, sink)
            e1.record()
            torch.cuda.synchronize()
            if rep >= 2:
                ts.append(e0.elapsed_time(e1) * 1e-3)
        ts.sort()
        res[name + "_G_per_s"] = n / ts[len(ts) // 2] / 1e9
    del table, sink
    return res


# ------------------------------------------------------------------------------------------------ CPU oracle
def host_copies(ctx, wl, with_features=True):
    """The workload's graph (and feature tables) as numpy arrays for the oracle."""
    import numpy as np

    import oracle as orc
    torch = ctx.torch
    to_np = lambda t: (t.view(torch.int16).cpu().numpy().view(np.uint16) if t.dtype == torch.bfloat16
                       else t.cpu().numpy())
    h = SimpleNamespace(orc=orc, np=np)
    h.indptr, h.indices = wl.indptr.cpu().numpy(), wl.indices.cpu().numpy()
    h.feats = to_np(wl.feats) if with_features else None
    if wl.requests is None:
        h.og = orc.Graph(h.indptr, h.indices)
        h.ofs = orc.FeatStore(h.feats) if with_features else None
    else:
        h.pos = wl.pos_map.cpu().numpy()
        h.og = orc.Graph(h.indptr, h.indices, row_begin=wl.lo, num_total_nodes=wl.N)
        h.ofs = orc.FeatStore(h.feats, to_np(wl.cache), h.pos) if with_features else None
        h.mv, h.rw = wl.min_vids.cpu().numpy(), wl.requests["remote_worker_map"].cpu().numpy()
    return h


def parity_of_batches(args, ctx, wl, h, pipe, seed_sets, keys, hops):
    """GPU pipeline against the oracle on the same seeds and rng keys, bit for bit: the node list, every hop's
    sampled ids, compact ids and counts, and the gathered rows (request lists and their bucket sizes for a
    partitioned store).  -> dict of what was compared; any mismatch makes `ok` false."""
    np, orc, torch = h.np, h.orc, ctx.torch
    out = {"batches": 0, "input_nodes": True, "neighbors": True, "relabeled": True, "counts": True,
           "features": True if h.ofs is not None else None}
    if wl.requests is not None:
        out["request_lists"] = True
    for seeds, key in zip(seed_sets, keys):
        pipe.run(seeds, key)
        res = pipe.result()
        want_in, want_blocks = orc.sample_blocks(h.og, seeds.cpu().numpy(), hops, args.replace, key)
        out["input_nodes"] &= bool(np.array_equal(res["input_nodes"].cpu().numpy(), want_in))
        for got, want in zip(res["blocks"], want_blocks):
            for k in ("neighbors", "relabeled", "counts"):
                out[k] &= bool(np.array_equal(got[k].cpu().numpy(), want[k]))
        rows_of = want_in
        if wl.requests is not None:
            bs, _, so, _ = orc.cluster_reqs(want_in, h.pos, h.rw, h.mv, wl.P, wl.P)
            out["request_lists"] &= (res["request_sizes"] == [int(x) for x in bs]
                                     and bool(np.array_equal(res["request_ids"].cpu().numpy(), so)))
            rows_of = so[:bs[0]]
        if h.ofs is not None:
            want_f, _ = orc.gather_rows(h.ofs, rows_of)
            got_f = res["features"]
            got_f = got_f.view(torch.int16).cpu().numpy().view(np.uint16) if got_f.dtype == torch.bfloat16 else got_f.cpu().numpy()
            out["features"] &= bool(np.array_equal(got_f, want_f))
        out["batches"] += 1
    out["ok"] = all(v for k, v in out.items() if k != "batches" and v is not None)
    return out


def stage_cpu_baseline(args, ctx, wl, m):
    """CPU baseline: the oracle on this machine's host cores on a bounded sample of the same workload, and the
    bit-for-bit comparison of the GPU's batches with the oracle's on the same host copies."""
    torch = ctx.torch
    budget = args.cpu_seconds
    h = host_copies(ctx, wl)
    np, orc = h.np, h.orc
    threads = args.cpu_threads or min(16, orc.max_threads())
    orc.set_threads(threads)
    K, W, hops = m.K, m.W, m.hops
    # parity first: the first two timed batches, rebuilt by the GPU pipeline and by the oracle
    keys = [args.seed + 100 + W + i for i in range(min(2, K))]
    parity = parity_of_batches(args, ctx, wl, h, m.stage_pipe, m.seed_sets[W:W + len(keys)], keys, hops)
    parity["what"] = (f"the first {len(keys)} timed batches rebuilt by the GPU pipeline and by the oracle on host copies "
                      f"of the same graph and feature table, compared bit for bit")
    h_seeds = [s.cpu().numpy() for s in m.seed_sets[W:]]

    def cpu_leg(seconds, first):
        """Batches of the timed seed sets (cycled with fresh rng keys) until `seconds` are used."""
        edges_done = batches = 0
        tc = 0.0
        while tc < seconds:
            s = h_seeds[(first + batches) % K]
            key = args.seed + 100 + W + first + batches
            t1 = time.perf_counter()
            inp, blocks = orc.sample_blocks(h.og, s, hops, args.replace, key)
            if wl.requests is None:
                orc.gather_rows(h.ofs, inp)
            else:
                bs, _, so, _ = orc.cluster_reqs(inp, h.pos, h.rw, h.mv, wl.P, wl.P)
                orc.gather_rows(h.ofs, so[:bs[0]])
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
    if wl.requests is None:
        inp, _ = orc.sample_blocks(h.og, h_seeds[0], hops, args.replace, args.seed + 100 + W)
        table = torch.from_numpy(h.feats.view(np.int16) if wl.dtype == torch.bfloat16 else h.feats)
        ids_t = torch.from_numpy(inp)
        torch.set_num_threads(threads)
        table.index_select(0, ids_t[:1000])
        t1 = time.perf_counter()
        reps = 0
        while time.perf_counter() - t1 < 1.0:
            table.index_select(0, ids_t)
            reps += 1
        tg = (time.perf_counter() - t1) / reps
        gather_cpu = dict(GBps=len(inp) * m.bytes_per_row / tg / 1e9, ms=tg * 1e3, rows=int(len(inp)),
                          what="torch.index_select on the host table (the reference's CPU gather), "
                               f"{threads} threads")
        del table, ids_t
    model = ""
    try:
        model = next(l.split(":", 1)[1].strip() for l in open("/proc/cpuinfo") if l.startswith("model name"))
    except (OSError, StopIteration):
        pass
    return dict(value=cpu_edges / tc, unit="edges/s", cores=threads, kind="port",
                sample=f"{cpu_batches} batches of the same workload (the timed seed sets, cycled "
                       f"with fresh rng keys) in {tc:.1f} s: sampling, relabel and gather on {threads} "
                       f"OpenMP threads",
                one_thread=one, gather_stage=gather_cpu, host_cpu=model, host_logical_cpus=os.cpu_count(),
                parity=parity)


# ------------------------------------------------------------------------------------------------ other configs
def stage_config(args, ctx, name, full_graph=None, with_aggregation=False):
    """One of the other configurations, measured like the main workload (fewer steps, no extras), its first
    batch checked against the oracle, then freed."""
    from bench_extra import stage_aggregation
    torch = ctx.torch
    w = dict(WORKLOADS[name])
    wl = build_workload(args, name, w, ctx, full_graph=full_graph)
    quiet_gc()
    hops = list(reversed(w["fan_out"]))
    K, W = args.config_steps, 10
    m = measure(args, ctx, wl, w["batch"], hops, K, W, event_steps=16, per_step=False, tag=f"{name}: ")
    tr = traffic_entry(MEASURED_GATHER_TRAFFIC_PER_ROW, args, wl, m.B)
    gq = quantiles([t * 1e3 for t in m.gather_ms]) if m.staged else None
    out = {
        "workload": f"{name}: {w['nodes']} nodes / {wl.num_edges_graph} directed edges held (max degree {wl.max_deg}), "
                    f"features {w['dim']} x {w['dtype']}, batch {w['batch']}, fan_out {w['fan_out']}" + wl.part_note,
        "graph": wl.graph_note, "steps": K, "warmup": W, "setup_s": wl.setup_s,
        "ms_per_step": m.elapsed / K * 1e3, "edges_per_s": m.edges_per_s, "edges_per_step": m.edges / K,
        "frontier_sizes_last_step": m.hop_sizes[-1], "request_bucket_sizes_last_step": m.request_sizes,
        "sample_relabel_ms": m.t_sample / K,
        "gather": {
            "rows": m.rows / K, "us_median": gq["median"] if gq else None, "us_p10": gq["p10"] if gq else None,
            "us_p90": gq["p90"] if gq else None, "us_mean": m.t_gather / K * 1e3,
            "bytes_per_row": m.bytes_per_row, "bytes_per_row_definition": m.bytes_per_row_def,
            "GBps": m.gather_gbps, "frac": m.gather_gbps / HBM_PEAK_GBPS,
            "frac_by_definition_bytes": m.gather_gbps / HBM_PEAK_GBPS * m.bytes_per_row_def / m.bytes_per_row,
            "traffic_bytes_per_row": tr[0] if tr else None, "traffic_source": tr[1] if tr else None,
        },
    }
    if args.inflight > 1 and args.driver == "fused":
        from apt_amd.loader import MiniBatchLoader
        loader = MiniBatchLoader(wl.graph, wl.store, torch.cat(m.seed_sets), m.B, hops, in_flight=args.inflight,
                                 shuffle=False, replace=args.replace, seed=args.seed, requests=wl.requests)
        t_ld, l_edges, gaps = time_loader(torch, loader, W)
        out["loader"] = {"batches_in_flight": args.inflight, "ms_per_step": t_ld / K * 1e3, "edges_per_s": l_edges / t_ld,
                         "ms_between_batches": gaps, "host_us_per_batch": loader_cost_per_batch(loader)}
        del loader
    if args.cpu_seconds > 0:
        h = host_copies(ctx, wl)      # the partition's two feature tables included (17 GB)
        h.orc.set_threads(args.cpu_threads or min(16, h.orc.max_threads()))
        out["parity"] = parity_of_batches(args, ctx, wl, h, m.stage_pipe, m.seed_sets[W:W + 1], [args.seed + 100 + W], hops)
        del h
    agg = None
    if with_aggregation:
        agg = stage_aggregation(ctx.capi, ctx.dev, ctx.synth, torch, m.stage_pipe, m.seed_sets[W + K - 1],
                                args.seed + 100 + W + K - 1, args.seed)
    ok = out.get("parity", {}).get("ok", True)
    del m, wl
    torch.cuda.empty_cache()
    return out, agg, ok


def main():
    args = parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU only (no collectives); use --gpus 1")
    if int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.exit("bench.py: launched with WORLD_SIZE > 1; this build runs on one GPU only")

    import torch

    import bench_extra as extra
    from apt_amd import capi, synth
    from apt_amd.pipeline import MiniBatchPipeline

    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    capi.lib()
    capi.bench_lib()
    for kv in filter(None, args.tune.split(",")):
        key, val = kv.split("=")
        capi.set_tuning(key, int(val))
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    ctx = SimpleNamespace(torch=torch, capi=capi, synth=synth, dev=dev, kev=KernelEvents(),
                          mark=TraceMarkers(torch, capi, dev))
    kev = ctx.kev

    w = dict(WORKLOADS[args.workload])
    if args.batch_size:
        w["batch"] = args.batch_size
    if args.feature_dtype:
        w["dtype"] = args.feature_dtype
    if args.fan_out:
        w["fan_out"] = [int(x) for x in args.fan_out.split(",")]
    hops = list(reversed(w["fan_out"]))            # reference python/npc/sampler.py:191
    B, K, W = w["batch"], args.steps, args.warmup
    H = len(hops)

    wl = build_workload(args, args.workload, w, ctx)
    quiet_gc()
    m = measure(args, ctx, wl, B, hops, K, W, args.event_steps)
    pipe, stage_pipe, seed_sets = m.pipe, m.stage_pipe, m.seed_sets
    edges, rows = m.edges, m.rows

    if args.calibration_copy_mib > 0:
        a = torch.ones(args.calibration_copy_mib << 20, dtype=torch.uint8, device=dev)
        b = torch.empty_like(a)
        capi.synth_copy(a, b)
        torch.cuda.synchronize()
        del a, b

    # ---- the same K batches with the relabel's last pass riding in the gather's launch
    # (MiniBatchPipeline(defer_lookup=True)): that launch is then no longer the gather alone, which is why
    # the timed region above, and with it `roofline`, keeps the pass as a launch of its own
    deferred = None
    if args.defer_lookup == "off" and args.driver == "fused" and wl.requests is None:
        dp = MiniBatchPipeline(wl.graph, wl.store, B, hops, replace=args.replace, defer_lookup=True)
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
            pipes.append(m.make_pipe(args.driver == "graph"))
            streams.append(torch.cuda.Stream())
        torch.cuda.synchronize()

        def run_batches(first, count):
            for i in range(count):
                k = i % len(pipes)
                with torch.cuda.stream(streams[k]):
                    pipes[k].run(seed_sets[first + i], args.seed + 100 + first + i)

        run_batches(0, W)
        ctx.mark(f"{K} batches, {len(pipes)} in flight on {len(pipes)} streams")
        t0 = time.perf_counter()
        run_batches(W, K)
        torch.cuda.synchronize()
        t_fl = time.perf_counter() - t0
        ctx.mark("end of the batches in flight")
        assert all(int(p.misses.item()) == 0 for p in pipes)
        in_flight = {"batches_in_flight": len(pipes), "ms_per_step": t_fl / K * 1e3,
                     "edges_per_s": edges / t_fl}
        if args.driver == "fused" and wl.requests is None:
            in_flight["timeline"] = extra.stage_in_flight_timeline(args, capi, kev, torch, pipes, streams, seed_sets,
                                                                   W, K, hops)
        del pipes[1:]
        # the same through the epoch loader a trainer would use (MiniBatchLoader): the consumer receives
        # every batch narrowed to its sizes, which costs one host read-back per batch
        if args.driver == "fused":
            from apt_amd.loader import MiniBatchLoader
            loader = MiniBatchLoader(wl.graph, wl.store, torch.cat(seed_sets), B, hops, in_flight=args.inflight,
                                     shuffle=False, replace=args.replace, seed=args.seed, requests=wl.requests)
            ctx.mark(f"epoch loader: {W} + {K} batches, {args.inflight} streams")
            t_ld, loader_edges, gaps = time_loader(torch, loader, W)
            ctx.mark("end of the epoch loader")
            in_flight["loader"] = {"ms_per_step": t_ld / K * 1e3, "edges_per_s": loader_edges / t_ld,
                                   "ms_between_batches": gaps, "host_us_per_batch": loader_cost_per_batch(loader)}
            del loader

    agg = None
    if args.aggregation:
        agg = extra.stage_aggregation(capi, dev, synth, torch, stage_pipe, seed_sets[W + K - 1],
                                      args.seed + 100 + W + K - 1, args.seed)
    fmt = None
    if args.formats:
        fmt = extra.stage_formats(args=args, B=B, graph=wl.graph, hops=hops, K=K, MiniBatchPipeline=MiniBatchPipeline,
                                  requests=wl.requests, seed_sets=seed_sets, store=wl.store, torch=torch, W=W,
                                  time_loader=time_loader)
    shuffle = None
    if args.shuffle:
        shuffle = extra.stage_shuffle(args=args, capi=capi, dev=dev, hops=hops, N=wl.N, seed_sets=seed_sets,
                                      stage_pipe=stage_pipe, torch=torch, W=W)
    cache_build = None
    if args.cache_build and wl.requests is None:
        cache_build = extra.stage_cache_build(args=args, B=B, bytes_per_row=m.bytes_per_row, capi=capi, dev=dev,
                                              graph=wl.graph, hops=hops, indptr=wl.indptr, N=wl.N,
                                              seed_sets=seed_sets, stage_pipe=stage_pipe, store=wl.store,
                                              torch=torch, W=W)

    # ---- CPU baseline: the oracle on this machine's host cores, bounded sample, and the parity check
    cpu = None
    parity_ok = True
    if args.cpu_seconds > 0:
        cpu = stage_cpu_baseline(args, ctx, wl, m)
        parity_ok = cpu["parity"]["ok"]

    # ---- the north-star sentence's own shape: batch 1024 on this graph, bf16 and fp32 rows
    target = None
    if args.target_leg == "on" or (args.target_leg == "auto" and args.workload == "full" and wl.requests is None):
        held = {}

        def store_of(name):
            want = torch.bfloat16 if name == "bf16" else torch.float32
            if wl.feats.dtype == want:
                return wl.store
            held.clear()                                  # one extra table at a time
            held[name] = synth.random_features(wl.N, w["dim"], want, args.seed + 1, dev)
            return capi.FeatStore(held[name])

        target = stage_target_shape(args, ctx, wl, hops, store_of)
        held.clear()
        torch.cuda.empty_cache()

    relabel_small = extra.stage_relabel_small(capi, dev, wl.N, torch) if args.relabel_small else None
    operators = None
    if args.operators and wl.requests is None and not args.replace:
        operators = extra.stage_operators(torch, wl, hops, seed_sets, W, K, args.seed + 5000)
    gather_sizes = None
    if args.gather_sizes and wl.requests is None:
        gather_sizes = extra.stage_gather_sizes(capi, dev, kev, wl.store, wl.N, torch)
    alternate = None
    if args.alternate and wl.requests is None:
        alternate = extra.stage_alternate(args, capi, wl.graph, hops, kev, MiniBatchPipeline, wl.seed_n, wl.seed_lo,
                                          wl.store, args.alternate_batch or B, torch, dev)

    # ---- what bounds the sampling kernel: random transactions.  The GPU's rate for them, measured here.
    ceilings = stage_ceilings(ctx, wl.N) if args.ceilings != "off" else None
    roofline_sampling = sampling_roofline(args, wl, m, ceilings)

    out = {
        "metric": "sampled edges/s (3-hop 15,10,5) + feature-gather GB/s as % of HBM peak",
        "value": m.edges_per_s,
        "unit": "edges/s",
        "n_gpus": 1,
        "steps": K,
        "warmup": W,
        "ms_per_step": m.elapsed / K * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int64",
        "data": "synthetic",
        "config": {
            "workload": f"{args.workload}: R-MAT {w['nodes']} nodes / {wl.num_edges_graph} directed edges "
                        f"(max degree {wl.max_deg}), features {w['dim']} x {w['dtype']}, batch {B}, "
                        f"fan_out {w['fan_out']} (hops from the seeds: {hops}), "
                        f"{'with' if args.replace else 'without'} replacement, relabel per hop, "
                        f"gather of all input nodes" + wl.part_note,
            "batch": B, "fan_out": w["fan_out"], "feature_dtype": w["dtype"], "driver": args.driver,
            "graph": wl.graph_note,
        },
        "roofline": gather_roofline(args, wl, m, pipe.can_defer_lookup),
        "roofline_sampling": roofline_sampling,
        "cpu_baseline": cpu,
        "aggregation": agg,
        "block_formats": fmt,
        "cache_build": cache_build,
        "shuffle": shuffle,
        "relabel_small": relabel_small,
        "operators": operators,
        "alternate": alternate,
        "gather_sizes": gather_sizes,
        "stages": {
            "target_shape": target,
            "per_step_ms": m.per_step_ms,
            "random_access_ceilings": ceilings,
            "in_flight": in_flight,
            "deferred_lookup": deferred,
            "edges_per_step": edges / K,
            "input_nodes_per_step": rows / K,
            "sample_relabel_ms": m.t_sample / K,
            "gather_ms": m.t_gather / K,
            "sample_relabel_edges_per_s": edges / (m.t_sample * 1e-3),
            "frontier_sizes_last_step": m.hop_sizes[-1],
            "request_bucket_sizes_last_step": m.request_sizes,
            "setup_s": wl.setup_s,
            "trace_markers": ctx.mark.names,
            "configs": None,
        },
    }

    # ---- the other configurations, one at a time, each freed before the next
    if args.configs == "on" or (args.configs == "auto" and args.workload == "full"):
        full_graph = (wl.indptr, wl.indices) if args.workload in ("full", "target") and args.graph == "symmetric" else None
        del m, pipe, stage_pipe, seed_sets
        wl.feats = wl.store = None                        # the main workload's feature table goes; its graph stays
        torch.cuda.empty_cache()
        configs = {}
        configs["partition"], agg5, ok = stage_config(args, ctx, "partition", full_graph=full_graph,
                                                      with_aggregation=True)
        parity_ok &= ok
        configs["aggregation"] = agg5
        del full_graph, wl
        torch.cuda.empty_cache()
        for name in ("medium", "small"):
            configs[name], _, ok = stage_config(args, ctx, name)
            parity_ok &= ok
        out["stages"]["configs"] = configs

    print(json.dumps(out))
    if not parity_ok:
        sys.exit("bench.py: the GPU's batches differ from the CPU oracle's (see cpu_baseline.parity and "
                 "stages.configs.*.parity in the line above)")


if __name__ == "__main__":
    main()
