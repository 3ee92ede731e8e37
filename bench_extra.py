"""Optional stages of bench.py (each behind a flag of its own): the aggregation kernels on a sampled
block, block formats, the local halves of the feature shuffle, cache construction, the gather kernel
at a range of launch sizes, the small-input relabel, and kernel-variant knobs compared inside one
process.  The default benchmark line needs none of them except the aggregation stage, which it runs
on the partition workload's block.  Every function takes what it needs from bench.py as arguments;
nothing here is imported by the library."""
import time

HBM_PEAK_GBPS = 8000.0


def quantiles(xs):
    """median / p10 / p90 / min / max of a list (nearest rank)."""
    v = sorted(xs)
    at = lambda q: v[min(len(v) - 1, max(0, int(round(q * (len(v) - 1)))))]
    return {"median": at(0.5), "p10": at(0.1), "p90": at(0.9), "min": v[0], "max": v[-1], "n": len(v)}


def gather_bytes_per_row(dim, esize, has_pos_map):
    """-> (bytes the launch moves per row, the per-row figure of the roofline definition).  Row read + row
    write + 8-byte id (+ the 8-byte position-map entry: the definition always counts it, the launch only reads
    it when the store has a map; an identity store has none)."""
    return 2 * dim * esize + 8 + (8 if has_pos_map else 0), 2 * dim * esize + 16


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


def stage_aggregation(capi, dev, synth, torch, pipe, seeds, rng_seed, data_seed=1):
    """The aggregation stage on the outermost block of one batch: GraphSAGE mean SpMM
    (hidden 256, fp32 and bf16 rows, fp32 accumulation) and a GAT layer of 4 heads x 64 (logits, then fused
    LeakyReLU + edge softmax + weighted sum), each with the bytes it has to move and its duration."""
    pipe.run(seeds, rng_seed)
    res = pipe.result()
    blk = res["blocks"][0]
    rel = blk["relabeled"]
    f = blk["fanout"]
    col_all = torch.arange(blk["seeds"].numel(), device=dev).repeat_interleave(f)
    keep = rel >= 0
    row_e, col_e = rel[keep].contiguous(), col_all[keep].contiguous()
    n_src, n_dst, E, hid = blk["unique"].numel(), blk["seeds"].numel(), int(keep.sum()), 256
    agg = {"edges": E, "num_src": n_src, "num_dst": n_dst, "hidden": hid, "fanout": f,
           "bytes": "SpMM mean: E x hidden x s read + num_dst x hidden x 4 written + 8 x num_dst x fanout of ids"}
    for name, dt, es in (("fp32", torch.float32, 4), ("bf16", torch.bfloat16, 2)):
        h = synth.random_features(n_src, hid, dt, data_seed + 7, dev)
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
        agg[f"spmm_block_mean_{name}_bytes"] = nbytes
        agg[f"spmm_block_mean_{name}_GBps"] = nbytes / t / 1e9
    # GAT layer of the same block: 4 heads x 64, logits then fused LeakyReLU + edge softmax + weighted sum
    heads, hdim = 4, 64
    for name, dt, es in (("fp32", torch.float32, 4), ("bf16", torch.bfloat16, 2)):
        ft = synth.random_features(n_src, heads * hdim, dt, data_seed + 9, dev).view(n_src, heads, hdim)
        al = (torch.randn(heads, hdim, device=dev) * 0.02).contiguous()
        ar = (torch.randn(heads, hdim, device=dev) * 0.02).contiguous()
        el, er = capi.gat_scores(ft, al), capi.gat_scores(ft[:n_dst], ar)
        for tag, fn, nbytes in (
                ("gat_scores", lambda: capi.gat_scores(ft, al), n_src * heads * (hdim * es + 4)),
                ("gat_block", lambda: capi.gat_block(rel, n_dst, f, ft, el, er, 0.2),
                 E * heads * (hdim * es + 4) + n_dst * heads * (hdim * 4 + 4) + 8 * n_dst * f)):
            t = seconds_per_call(torch, fn)
            agg[f"{tag}_{name}_us"] = t * 1e6
            agg[f"{tag}_{name}_bytes"] = nbytes
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
    hd = synth.random_features(n_dst, hid, torch.float32, data_seed + 8, dev)
    h = synth.random_features(n_src, hid, torch.float32, data_seed + 7, dev)
    fn = lambda: capi.sddmm(0, row_e, col_e, h, hd)
    t = seconds_per_call(torch, fn)
    agg["sddmm_u_add_v_fp32_us"] = t * 1e6
    agg["sddmm_u_add_v_fp32_GBps"] = (3 * E * hid * 4 + 16 * E) / t / 1e9
    del h, hd
    return agg


def stage_formats(args, B, graph, hops, K, MiniBatchPipeline, requests, seed_sets, store, torch, W, time_loader=None):
    """Every hop's block as COO + CSC (+ CSR of all blocks, or of all but the outermost), device-side sizes, after
    sampling."""
    ev = lambda: torch.cuda.Event(enable_timing=True)
    fmt = {}
    for name, what in (("coo_csc", "csc"), ("coo_csc_csr_inner", "inner"), ("coo_csc_csr", True)):
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
        if time_loader is not None and args.inflight > 1:
            # what a trainer receives: the epoch loader with the formats in every batch, through the library's
            # epoch thread and through the Python driver
            from apt_amd.loader import MiniBatchLoader
            for drv in ("c", "python"):
                ld = MiniBatchLoader(graph, store, torch.cat(seed_sets), B, hops, in_flight=args.inflight, shuffle=False,
                                     replace=args.replace, seed=args.seed, requests=requests, formats=what, driver=drv)
                t_ld, _, _ = time_loader(torch, ld, W)
                fmt[f"{name}_loader_{drv}_ms"] = t_ld / K * 1e3
                del ld
    return fmt


def stage_shuffle(args, capi, dev, hops, N, seed_sets, stage_pipe, torch, W):
    """Bucketing by owner and pack / unpack of hidden rows (the local halves of feat_shuffle)."""
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
    """Cache construction and the strategy dry run (the callers of the registries)."""
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


TUNING_DEFAULTS = {"minibatch_fuse_mark": 1, "relabel_lds": 1, "block_fused_scan": 1}


def stage_operators(torch, wl, hops, seed_sets, W, K, rng_base):
    """The batch through the operator layer (torch.ops.npc.*), as the reference's sampler calls it
    (python/npc/sampler.py:187-203): local_sample_one_layer + relabel_csc per hop, with the rank table of the
    registered graph and with the hash table; then the one operator that runs all hops (sample_blocks), with
    fresh output tensors per call (the default) and with the ring of two buffer sets.  No gather; every call
    returns narrowed tensors, i.e. reads its sizes back as the reference's operators do."""
    import apt_amd as npc
    empty = torch.empty(0, dtype=torch.int64)
    npc.set_topology(0, 1)
    npc.mix_cache_graphs(0, empty, empty, empty, wl.indptr, wl.indices)
    n = min(K, 60)

    def per_hop(seeds, key):
        frontier = seeds
        for h, f in enumerate(hops):
            nb, _ = npc.ops.sample_neighbors(frontier, f, False, key, h)
            frontier, _ = npc.ops.tensor_relabel_csc(frontier, nb)
        return frontier

    def timed(fn):
        for i in range(min(W, 10)):
            fn(seed_sets[i], rng_base + i)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(n):
            fn(seed_sets[W + i], rng_base + W + i)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / n * 1e3

    out = {"batches": n}
    try:
        npc.ops.set_ranked_relabel(True)
        out["per_hop_rank_table_ms"] = timed(per_hop)
        npc.ops.set_ranked_relabel(False)
        out["per_hop_hash_table_ms"] = timed(per_hop)
        npc.ops.set_ranked_relabel(True)
        blocks = lambda seeds, key: npc.ops.sample_blocks(seeds, list(hops), False, key)
        out["sample_blocks_fresh_tensors_ms"] = timed(blocks)
        npc.ops.set_block_buffer_ring(2)
        out["sample_blocks_ring_of_two_ms"] = timed(blocks)
    finally:
        npc.ops.set_block_buffer_ring(0)
        npc.ops.set_ranked_relabel(True)
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
    default_of = lambda k: TUNING_DEFAULTS.get(k, 0)
    H, NB = len(hops), 40
    pipe = MiniBatchPipeline(graph, store, B, hops, replace=args.replace, fused=not args.driver.startswith("unfused"),
                             relabel="hash" if args.driver == "unfused_hash" else "ranked")
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


def interval_union(iv):
    """Total length covered by a list of (start, end) intervals."""
    tot, cs, ce = 0.0, None, None
    for s_, e_ in sorted(iv):
        if cs is None:
            cs, ce = s_, e_
        elif s_ > ce:
            tot += ce - cs
            cs, ce = s_, e_
        else:
            ce = max(ce, e_)
    return tot + (ce - cs if cs is not None else 0.0)


def covered_at_least(iv, k):
    """Total time during which at least k of the intervals are open."""
    pts = sorted([(s_, 1) for s_, _ in iv] + [(e_, -1) for _, e_ in iv])
    tot, open_, last = 0.0, 0, None
    for t, d in pts:
        if last is not None and open_ >= k:
            tot += t - last
        open_ += d
        last = t
    return tot


def stage_in_flight_timeline(args, capi, kev, torch, pipes, streams, seed_sets, first, count, hops):
    """Where the time of the batches-in-flight arrangement goes, without a profiler in the way: every batch's
    last-hop sampling kernel and gather kernel carry HIP events on their dispatches; read against one base
    event they give each kernel's begin and end on the GPU's clock, across streams.  -> how much of the
    region has a gather running, a last-hop sampler running, two of a kind at once, one of each at once, or
    neither (only the short kernels of hops 1-2 and the relabel passes), and how the two kernels stretch when
    they share the GPU."""
    H = len(hops)
    base = kev.pair()
    gp, sp = [], []
    torch.cuda.synchronize()
    kev.record(base[0], streams[0])
    for i in range(count):
        k = i % len(pipes)
        with torch.cuda.stream(streams[k]):
            g, s_ = kev.pair(), kev.pair()
            capi.check(capi.lib().apt_time_next_sample(H - 1, s_[0], s_[1]))
            pipes[k].sample(seed_sets[first + i], args.seed + 100 + first + i, defer_lookup=True)
            capi.check(capi.lib().apt_time_next_gather(g[0], g[1]))
            pipes[k].gather()
            gp.append(g)
            sp.append(s_)
    torch.cuda.synchronize()
    at = lambda ev: kev.ms((base[0], ev), destroy=False) * 1e3
    gat = [(at(a), at(b)) for a, b in gp]
    sam = [(at(a), at(b)) for a, b in sp]
    for pr in gp + sp + [base]:
        kev.destroy(pr)
    # leave the ramp-up and the drain out: the middle 80 % of the batches
    lo, hi = count // 10, count - count // 10
    gat_m, sam_m = gat[lo:hi], sam[lo:hi]
    t0, t1 = min(s_ for s_, _ in sam_m), max(e_ for _, e_ in gat_m)
    clip = lambda iv: [(max(a, t0), min(b, t1)) for a, b in iv if b > t0 and a < t1]
    g_all, s_all = clip(gat), clip(sam)
    span = t1 - t0
    both = interval_union(g_all) + interval_union(s_all) - interval_union(g_all + s_all)
    return {
        "batches": hi - lo, "us_per_batch": span / (hi - lo),
        "gather_us_mean": sum(b - a for a, b in gat_m) / len(gat_m),
        "last_hop_sample_us_mean": sum(b - a for a, b in sam_m) / len(sam_m),
        "fraction_of_time": {
            "a_gather_running": interval_union(g_all) / span,
            "a_last_hop_sampler_running": interval_union(s_all) / span,
            "either_running": interval_union(g_all + s_all) / span,
            "a_gather_and_a_sampler_running": both / span,
            "two_or_more_gathers_running": covered_at_least(g_all, 2) / span,
            "two_or_more_samplers_running": covered_at_least(s_all, 2) / span,
            "neither_running": 1.0 - interval_union(g_all + s_all) / span,
        },
        "timing": "HIP events carried by every batch's two largest dispatches, read against one base event",
    }
