"""The pipeline at the benchmark's sizes.

medium (2.4 M nodes / 62 M edges): the graph is copied to the host and the
whole batch is compared with the oracle, bit for bit.
full (111 M nodes, 1.6 B R-MAT edges stored in both directions plus a self-loop
per node, 128 x bf16): the graph (27 GB) is copied to the host once and whole
batches of 4096 seeds are compared with the oracle bit for bit, with and
without replacement; the gathered rows are compared with torch's own
index_select of the same ids (the 28 GB feature table stays on the GPU).  The
properties that hold at any size are checked as well: counts = min(fanout,
degree), sampled ids are true neighbours, the node list has no duplicates and
starts with the seeds, nodes[relabeled] gives the sampled ids back, and the same
rng key reproduces the batch.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _check_properties(pipe, graph_t, feats, seeds, hops, replace):
    indptr, indices = graph_t
    res = pipe.result()
    nodes = res["input_nodes"]
    B = seeds.numel()
    assert torch.equal(nodes[:B], seeds)                                    # dst nodes are a prefix of src nodes
    assert torch.unique(nodes).numel() == nodes.numel()                     # no duplicates
    total = 0
    for h, blk in enumerate(reversed(res["blocks"])):
        f = blk["fanout"]
        front = blk["seeds"]
        deg = indptr[front + 1] - indptr[front]
        want_cnt = torch.where(deg > 0, torch.full_like(deg, f), torch.zeros_like(deg)) if replace \
            else torch.minimum(deg, torch.full_like(deg, f))
        assert torch.equal(blk["counts"], want_cnt)
        nbr = blk["neighbors"].view(-1, f)
        rel = blk["relabeled"].view(-1, f)
        valid = torch.arange(f, device=DEV)[None, :] < blk["counts"][:, None]
        assert torch.equal(nbr >= 0, valid) and torch.equal(rel >= 0, valid)
        assert torch.equal(blk["unique"][rel[valid]], nbr[valid])           # relabel round trip
        assert int(rel.max()) < blk["unique"].numel()
        total += int(blk["counts"].sum())
        # rows that fit in the fanout come back whole, in CSR order
        if not replace:
            small = torch.nonzero((deg > 0) & (deg <= f)).flatten()[:2000]
            for r in small[:200].tolist():
                s, e = int(indptr[front[r]]), int(indptr[front[r] + 1])
                assert torch.equal(nbr[r, :e - s], indices[s:e])
        # a sample of the other rows: every id is a neighbour; without replacement no position twice
        big = torch.nonzero(deg > f).flatten()
        pick = big[torch.randperm(big.numel(), device=DEV)[:100]]
        for r in pick.tolist():
            s, e = int(indptr[front[r]]), int(indptr[front[r] + 1])
            row = indices[s:e]
            got = nbr[r]
            assert bool(torch.isin(got, row).all())
            if not replace:
                # multiset containment: an id may repeat in a multigraph row, but not more often than it occurs
                vals, cnts = torch.unique(got, return_counts=True)
                for v, c in zip(vals.tolist(), cnts.tolist()):
                    assert int((row == v).sum()) >= c
    assert total == res["num_edges"]
    if feats is not None:
        assert torch.equal(res["features"].view(torch.int16) if feats.dtype == torch.bfloat16 else res["features"],
                           (feats.index_select(0, nodes).view(torch.int16) if feats.dtype == torch.bfloat16
                            else feats.index_select(0, nodes)))
    return res


def _check_formats(blk):
    """COO / CSC / CSR of a block against the fixed-stride layout they come from."""
    f, fmt = blk["fanout"], blk["formats"]
    rel = blk["relabeled"].view(-1, f)
    num_dst, num_src, E = rel.shape[0], blk["unique"].numel(), fmt["num_edges"]
    valid = rel >= 0
    assert E == int(valid.sum())
    assert torch.equal(fmt["coo_row"], rel[valid])                                   # destination-major order
    assert torch.equal(fmt["coo_col"], torch.arange(num_dst, device=DEV)[:, None].expand(-1, f)[valid])
    want = torch.zeros(num_dst + 1, dtype=torch.int64, device=DEV)
    want[1:] = torch.cumsum(valid.sum(1), 0)
    assert torch.equal(fmt["csc_indptr"], want)
    eids, ip = fmt["csr_eids"], fmt["csr_indptr"]
    assert ip.numel() == num_src + 1 and int(ip[0]) == 0 and int(ip[-1]) == E
    assert torch.equal(torch.sort(eids).values, torch.arange(E, device=DEV))         # a permutation of the edges
    src = fmt["coo_row"][eids]
    assert torch.equal(src, torch.repeat_interleave(torch.arange(num_src, device=DEV), ip[1:] - ip[:-1]))
    assert torch.equal(fmt["csr_indices"], fmt["coo_col"][eids])
    assert bool(((eids[1:] > eids[:-1]) | (src[1:] != src[:-1])).all())              # stable inside a source


def test_medium_scale_vs_oracle(orc, capi):
    from apt_amd import synth
    from apt_amd.pipeline import MiniBatchPipeline
    N, E, D = 2_449_029, 62_000_000, 100
    indptr, indices = synth.rmat_symmetric_csr_gpu(N, E, 1, DEV)
    feats = synth.random_features(N, D, torch.float32, 2, DEV)
    graph, store = capi.Graph(indptr, indices), capi.FeatStore(feats)
    hops = [5, 10, 15]
    pipe = MiniBatchPipeline(graph, store, 1024, hops, replace=False)
    og = orc.Graph(indptr.cpu().numpy(), indices.cpu().numpy())
    ofs = orc.FeatStore(feats.cpu().numpy())
    orc.set_threads(16)
    gen = torch.Generator(device=DEV)
    gen.manual_seed(3)
    for batch in range(3):
        seeds = torch.randperm(N, generator=gen, device=DEV)[:1024].contiguous()
        pipe.run(seeds, 77 + batch)
        res = _check_properties(pipe, (indptr, indices), feats, seeds, hops, False)
        want_in, want_blocks = orc.sample_blocks(og, seeds.cpu().numpy(), hops, False, 77 + batch)
        assert np.array_equal(res["input_nodes"].cpu().numpy(), want_in)
        for got, want in zip(res["blocks"], want_blocks):
            for k in ("neighbors", "relabeled", "counts"):
                assert np.array_equal(got[k].cpu().numpy(), want[k]), k
        want_f, _ = orc.gather_rows(ofs, want_in)
        assert np.array_equal(res["features"].cpu().numpy(), want_f)
    orc.set_threads(1)


FULL_N, FULL_E, FULL_D = 111_059_956, 3_200_000_000, 128


@pytest.fixture(scope="module")
def full(capi):
    """The full-scale graph and feature table, built once for this module and freed after it."""
    from apt_amd import synth
    stats = {}
    indptr, indices = synth.rmat_symmetric_csr_gpu(FULL_N, FULL_E, 1, DEV, stats=stats)
    feats = synth.random_features(FULL_N, FULL_D, torch.bfloat16, 2, DEV)
    box = dict(indptr=indptr, indices=indices, feats=feats, stats=stats)
    yield box
    box.clear()
    del indptr, indices, feats
    torch.cuda.empty_cache()


def test_full_scale_graph_is_simple_symmetric_with_self_loops(full):
    """What the generator promises (the kind of graph the reference trains on, scripts/load_data.py:13-17),
    checked at full size with size-independent properties and on sampled rows."""
    indptr, indices, st = full["indptr"], full["indices"], full["stats"]
    N = FULL_N
    assert indptr.numel() == N + 1 and int(indptr[0]) == 0 and int(indptr[-1]) == indices.numel()
    assert st["forward_edges"] > 1_550_000_000 and st["entries_before_merge"] == 2 * st["forward_edges"] + N
    assert indices.numel() > 2_800_000_000                           # what is left after merging repeats
    deg = indptr[1:] - indptr[:-1]
    assert int(deg.min()) >= 1                                       # every node has at least its self-loop
    assert int(indices.min()) >= 0 and int(indices.max()) < N
    # rows strictly increasing (sorted, no repeats): a decrease is only allowed where a new row starts
    step = 1 << 28
    row_start = torch.zeros(indices.numel(), dtype=torch.bool, device=DEV)
    row_start[indptr[:-1]] = True
    for s in range(0, indices.numel() - 1, step):
        e = min(s + step, indices.numel() - 1)
        assert bool(((indices[s + 1:e + 1] > indices[s:e]) | row_start[s + 1:e + 1]).all())
    del row_start
    gen = torch.Generator(device=DEV)
    gen.manual_seed(1)
    rows = torch.cat([torch.randint(0, N, (300,), generator=gen, device=DEV), torch.topk(deg, 3).indices]).tolist()
    for u in rows:
        row = indices[int(indptr[u]):int(indptr[u + 1])]
        assert bool((row == u).any())                                # the self-loop
        for v in row[torch.randperm(row.numel(), device=DEV)[:20]].tolist():   # symmetry: u in row v
            rv = indices[int(indptr[v]):int(indptr[v + 1])]
            k = int(torch.searchsorted(rv, torch.tensor(u, device=DEV)))
            assert k < rv.numel() and int(rv[k]) == u
    # every entry (u, v) has its mirror image (v, u): then the sum of u * v^2 over all entries equals the sum
    # of v * u^2 (64-bit wrap-around, an odd multiplier mixed in); over the entries with both ends among the
    # first million nodes, which hold the hubs
    M = 1 << 20
    src = torch.repeat_interleave(torch.arange(M, device=DEV), deg[:M])
    sub = indices[:src.numel()]
    inside = sub < M
    a, b = src[inside], sub[inside]
    assert a.numel() > 10_000_000
    h = 0x9E3779B97F4A7C15 - (1 << 64)
    assert int((a * (b * b * h)).sum()) == int((b * (a * a * h)).sum())
    assert int((a * (b * b * h)).sum()) != int(((a + 1) * (b * b * h)).sum())


def test_full_scale_vs_oracle(orc, capi, full):
    """Whole batches of 4096 seeds on the full-scale graph against the CPU oracle, bit for bit: the node list
    and every hop's sampled ids, compact ids and counts, without and with replacement, fused driver and
    per-hop driver; gathered rows against index_select."""
    from apt_amd.pipeline import MiniBatchPipeline
    indptr, indices, feats = full["indptr"], full["indices"], full["feats"]
    graph, store = capi.Graph(indptr, indices), capi.FeatStore(feats)
    og = orc.Graph(indptr.cpu().numpy(), indices.cpu().numpy())
    orc.set_threads(16)
    hops = [5, 10, 15]
    gen = torch.Generator(device=DEV)
    gen.manual_seed(11)
    try:
        for replace in (False, True):
            pipes = [MiniBatchPipeline(graph, store, 4096, hops, replace=replace),
                     MiniBatchPipeline(graph, None, 4096, hops, replace=replace, gather=False, fused=False),
                     MiniBatchPipeline(graph, None, 4096, hops, replace=replace, gather=False, fused=False,
                                       relabel="ranked_bidding")]
            for batch in range(2):
                seeds = torch.randperm(FULL_N, generator=gen, device=DEV)[:4096].contiguous()
                key = 31337 + 10 * batch + int(replace)
                want_in, want_blocks = orc.sample_blocks(og, seeds.cpu().numpy(), hops, replace, key)
                assert sum(int(b["counts"].sum()) for b in want_blocks) > 500_000
                for pipe in pipes[:1 if batch else 3]:
                    pipe.run(seeds, key)
                    res = pipe.result()
                    assert np.array_equal(res["input_nodes"].cpu().numpy(), want_in)
                    for got, want in zip(res["blocks"], want_blocks):
                        for k in ("neighbors", "relabeled", "counts"):
                            assert np.array_equal(got[k].cpu().numpy(), want[k]), (k, replace, batch)
                    if res["features"] is not None:
                        ids = torch.from_numpy(want_in).to(DEV)
                        assert torch.equal(res["features"].view(torch.int16), feats.index_select(0, ids).view(torch.int16))
            del pipes
    finally:
        orc.set_threads(1)
        del og


@pytest.mark.parametrize("replace", [False, True])
def test_full_scale_properties(capi, full, replace):
    from apt_amd.pipeline import MiniBatchPipeline
    N = FULL_N
    indptr, indices, feats = full["indptr"], full["indices"], full["feats"]
    graph, store = capi.Graph(indptr, indices), capi.FeatStore(feats)
    hops = [5, 10, 15]
    pipe = MiniBatchPipeline(graph, store, 4096, hops, replace=replace, formats=True)
    gen = torch.Generator(device=DEV)
    gen.manual_seed(5)
    seeds = torch.randperm(N, generator=gen, device=DEV)[:4096].contiguous()
    pipe.run(seeds, 2025)
    res = _check_properties(pipe, (indptr, indices), feats, seeds, hops, replace)
    for blk in res["blocks"]:
        _check_formats(blk)
    first = {k: res[k].clone() for k in ("input_nodes", "features")}
    rel0 = [b["relabeled"].clone() for b in res["blocks"]]
    # the same key reproduces the batch (also after other batches went through the rank table)
    pipe.run(torch.randperm(N, generator=gen, device=DEV)[:4096].contiguous(), 1)
    pipe.result()
    pipe.run(seeds, 2025)
    again = pipe.result()
    assert torch.equal(again["input_nodes"], first["input_nodes"])
    assert torch.equal(again["features"].view(torch.int16), first["features"].view(torch.int16))
    for a, b in zip(again["blocks"], rel0):
        assert torch.equal(a["relabeled"], b)
    # a different key samples differently
    pipe.run(seeds, 2026)
    assert not torch.equal(pipe.result()["input_nodes"], first["input_nodes"])
    if not replace:
        # the million highest-degree rows in a second CSR built on the GPU: same offsets as the degrees say,
        # and sampling through it (cached rows from the copy, the rest from the main table) changes nothing
        deg = indptr[1:] - indptr[:-1]
        hot = torch.topk(deg, 1_000_000).indices.contiguous()
        c_indptr, c_indices = capi.csr_select_rows(graph, hot)
        assert torch.equal(c_indptr[1:], torch.cumsum(deg[hot], 0)) and c_indices.numel() == int(c_indptr[-1])
        hub = int(hot[0])                                              # the 2 M-edge hub row, copied by many workgroups
        assert torch.equal(c_indices[:int(c_indptr[1])], indices[int(indptr[hub]):int(indptr[hub + 1])])
        k = int(torch.randint(1, 1_000_000, (1,)))
        assert torch.equal(c_indices[int(c_indptr[k]):int(c_indptr[k + 1])],
                           indices[int(indptr[hot[k]]):int(indptr[hot[k] + 1])])
        pos = -torch.arange(N, dtype=torch.int64, device=DEV) - 2
        pos[hot] = torch.arange(hot.numel(), device=DEV)
        cached_graph = capi.Graph(indptr, indices, cached_indptr=c_indptr, cached_indices=c_indices, adj_pos_map=pos)
        frontier = torch.cat([hot[:20000], torch.randint(0, N, (50000,), generator=gen, device=DEV)])
        a = capi.sample_neighbors(graph, frontier, 15, False, 99, 2)
        b = capi.sample_neighbors(cached_graph, frontier, 15, False, 99, 2)
        assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
        del pos, c_indptr, c_indices
        # an epoch of 1300 batches through the loader, two in flight: each pipeline's rank table runs out of
        # epochs once on the way (511 per fill at this plan's id width) and is refilled; every 40th batch is
        # rebuilt afterwards by a lone pipeline from the same seeds and key and must match bit for bit
        from apt_amd.loader import MiniBatchLoader
        ids = torch.randperm(N, generator=gen, device=DEV)[:1300 * 4096].contiguous()
        loader = MiniBatchLoader(graph, store, ids, 4096, hops, in_flight=2, shuffle=False, seed=3)
        kept, edges = {}, 0
        for i, batch in enumerate(loader):
            edges += batch["num_edges"]
            if i % 40 == 0:
                kept[i] = (batch["input_nodes"].clone(), batch["features"].view(torch.int16).clone(),
                           batch["blocks"][0]["relabeled"].clone())
        assert i == 1299 and edges > 1300 * 1_000_000
        for i, (nodes_i, feats_i, rel_i) in kept.items():
            pipe.run(ids[i * 4096:(i + 1) * 4096], 3 * 7919 * 1300 + i)
            want = pipe.result()
            assert torch.equal(want["input_nodes"], nodes_i), i
            assert torch.equal(want["features"].view(torch.int16), feats_i), i
            assert torch.equal(want["blocks"][0]["relabeled"], rel_i), i
        del loader, kept
    del pipe
    torch.cuda.empty_cache()


def test_fused_and_per_hop_drivers_agree_over_many_batches(capi):
    """Three hundred batches on the 2.4 M-node graph: the fused driver (rank table, bids inside
    the sampling kernel), the per-hop driver with the hash table and the per-hop driver with the rank
    table (apt_relabel_ranked, later hops continuing the batch; its 8-bit epoch field runs out and the
    table is refilled on the way) are three implementations of the same first-occurrence relabel and
    must agree bit for bit, whatever the scheduling of a batch was."""
    from apt_amd import synth
    from apt_amd.pipeline import MiniBatchPipeline
    N = 2_400_000
    indptr, indices = synth.rmat_csr_gpu(N, 62_000_000, 4, DEV)
    graph = capi.Graph(indptr, indices)
    hops = [5, 10, 15]
    fused = MiniBatchPipeline(graph, None, 1024, hops, gather=False)
    per_hop = MiniBatchPipeline(graph, None, 1024, hops, gather=False, fused=False)
    ranked = MiniBatchPipeline(graph, None, 1024, hops, gather=False, fused=False, relabel="ranked")
    # ... and the same with the bids placed by each hop's sampling call (apt_sample_neighbors_bidding)
    bidding = MiniBatchPipeline(graph, None, 1024, hops, gather=False, fused=False, relabel="ranked_bidding")
    gen = torch.Generator(device=DEV)
    gen.manual_seed(21)
    for batch in range(300):
        seeds = torch.randint(0, N, (1024,), generator=gen, device=DEV)          # repeated seeds happen
        fused.run(seeds, 9000 + batch)
        per_hop.run(seeds, 9000 + batch)
        ranked.run(seeds, 9000 + batch)
        bidding.run(seeds, 9000 + batch)
        a = fused.result()
        for other in (per_hop, ranked, bidding):
            b = other.result()
            assert a["sizes"] == b["sizes"], batch
            assert torch.equal(a["input_nodes"], b["input_nodes"]), batch
            for x, y in zip(a["blocks"], b["blocks"]):
                assert torch.equal(x["relabeled"], y["relabeled"]) and torch.equal(x["neighbors"], y["neighbors"]), batch
        assert int(ranked.ranked_outside) == 0 and int(bidding.ranked_outside) == 0
