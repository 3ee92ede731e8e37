"""The pipeline at the benchmark's sizes.

medium (2.4 M nodes / 62 M edges): the graph is copied to the host and the
whole batch is compared with the oracle, bit for bit.
full (111 M nodes / 3.2 B edges, 128 x bf16): too big to hand to the CPU oracle
in a test, so the batch is checked through properties that do not depend on
size: counts = min(fanout, degree), sampled ids are true neighbours, the node
list has no duplicates and starts with the seeds, nodes[relabeled] gives the
sampled ids back, the gathered rows equal torch's own index_select, and the
same rng key reproduces the batch.
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
    indptr, indices = synth.rmat_csr_gpu(N, E, 1, DEV)
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


@pytest.mark.parametrize("replace", [False, True])
def test_full_scale_properties(capi, replace):
    from apt_amd import synth
    from apt_amd.pipeline import MiniBatchPipeline
    N, E, D = 111_059_956, 3_200_000_000, 128
    indptr, indices = synth.rmat_csr_gpu(N, E, 1, DEV)
    assert indices.numel() > 3_000_000_000 and int(indptr[-1]) == indices.numel()
    feats = synth.random_features(N, D, torch.bfloat16, 2, DEV)
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
    del pipe, feats, indices, indptr
    torch.cuda.empty_cache()


def test_fused_and_per_hop_drivers_agree_over_many_batches(capi):
    """Three hundred batches on the 2.4 M-node graph: the fused driver (rank table, bids inside
    the sampling kernel) and the per-hop driver (hash table) are two implementations of the same
    first-occurrence relabel and must agree bit for bit, whatever the scheduling of a batch was."""
    from apt_amd import synth
    from apt_amd.pipeline import MiniBatchPipeline
    N = 2_400_000
    indptr, indices = synth.rmat_csr_gpu(N, 62_000_000, 4, DEV)
    graph = capi.Graph(indptr, indices)
    hops = [5, 10, 15]
    fused = MiniBatchPipeline(graph, None, 1024, hops, gather=False)
    per_hop = MiniBatchPipeline(graph, None, 1024, hops, gather=False, fused=False)
    gen = torch.Generator(device=DEV)
    gen.manual_seed(21)
    for batch in range(300):
        seeds = torch.randint(0, N, (1024,), generator=gen, device=DEV)          # repeated seeds happen
        fused.run(seeds, 9000 + batch)
        per_hop.run(seeds, 9000 + batch)
        a, b = fused.result(), per_hop.result()
        assert a["sizes"] == b["sizes"], batch
        assert torch.equal(a["input_nodes"], b["input_nodes"]), batch
        for x, y in zip(a["blocks"], b["blocks"]):
            assert torch.equal(x["relabeled"], y["relabeled"]) and torch.equal(x["neighbors"], y["neighbors"]), batch
