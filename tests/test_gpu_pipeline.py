"""The fused multi-hop pipeline and the operator layer vs the oracle's driver."""
import numpy as np
import pytest
import torch

from helpers import small_graph

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def _setup(orc, capi, n=30000, deg=14, dim=100, seed=21):
    indptr, indices = small_graph(n, deg, seed=seed)
    feats = np.random.default_rng(seed).standard_normal((n, dim)).astype(np.float32)
    return indptr, indices, feats


@pytest.mark.parametrize("mode", ["fused", "graph", "unfused", "unfused_ranked", "unfused_ranked_bidding"])
@pytest.mark.parametrize("replace", [False, True])
def test_pipeline_matches_oracle_driver(orc, capi, replace, mode):
    from apt_amd.pipeline import MiniBatchPipeline
    indptr, indices, feats = _setup(orc, capi)
    og = orc.Graph(indptr, indices)
    dg = capi.Graph(dev(indptr), dev(indices))
    fs = capi.FeatStore(dev(feats))
    hops = [5, 10, 15]
    pipe = MiniBatchPipeline(dg, fs, 512, hops, replace=replace, fused=not mode.startswith("unfused"),
                             use_graph=mode == "graph", relabel=mode[len("unfused_"):] or "hash")
    rng = np.random.default_rng(0)
    for batch in range(4):                                   # buffers (and the graph) are reused
        seeds = rng.permutation(len(indptr) - 1)[:512]
        if batch == 2:
            seeds[100:200] = seeds[0:100]                    # repeated seeds are legal
        pipe.run(dev(seeds), 1000 + batch)
        res = pipe.result()
        want_in, want_blocks = orc.sample_blocks(og, seeds, hops, replace, 1000 + batch)
        assert np.array_equal(res["input_nodes"].cpu().numpy(), want_in)
        for got, want in zip(res["blocks"], want_blocks):
            for k in ("seeds", "neighbors", "relabeled", "counts", "unique"):
                assert np.array_equal(got[k].cpu().numpy(), want[k]), k
        assert res["num_edges"] == sum(int(b["counts"].sum()) for b in want_blocks)
        want_f, miss = orc.gather_rows(orc.FeatStore(feats), want_in)
        assert miss == 0 and int(pipe.misses.item()) == 0
        assert np.array_equal(res["features"].cpu().numpy(), want_f)
        # structure (reference sampler.py:358-364): dst nodes are a prefix of src nodes
        if batch != 2:
            assert np.array_equal(want_in[:512], seeds)


def test_fused_driver_edge_cases(orc, capi):
    from apt_amd.pipeline import MiniBatchPipeline
    from helpers import special_graph
    indptr, indices, degs = special_graph()
    og = orc.Graph(indptr, indices)
    dg = capi.Graph(dev(indptr), dev(indices))
    for hops, replace in [([5], False), ([16, 3], False), ([2, 2, 2, 2], True), ([64], False)]:
        seeds = np.array([0, 1, 2, 3, 4, 5, 6, 6, 7, 8, 9, 10, 11, 5, -1, 3])
        pipe = MiniBatchPipeline(dg, None, len(seeds), hops, replace=replace, gather=False)
        pipe.run(dev(seeds), 77)
        res = pipe.result()
        want_in, want_blocks = orc.sample_blocks(og, seeds, hops, replace, 77)
        assert np.array_equal(res["input_nodes"].cpu().numpy(), want_in)
        for got, want in zip(res["blocks"], want_blocks):
            for k in ("neighbors", "relabeled", "counts", "unique"):
                assert np.array_equal(got[k].cpu().numpy(), want[k]), (hops, k)


def test_operator_layer_dp_sampler(orc, capi):
    import apt_amd as npc
    indptr, indices, feats = _setup(orc, capi, n=8000, dim=32, seed=5)
    n = len(indptr) - 1
    npc.set_topology(0, 1)
    e = torch.empty(0, dtype=torch.int64)
    npc.mix_cache_graphs(0, e, e, e, torch.from_numpy(indptr), torch.from_numpy(indices))
    npc.cache_feats_shared(n, torch.from_numpy(feats), torch.empty(0, 32), e, torch.arange(n), 0)
    og = orc.Graph(indptr, indices)
    seeds = np.random.default_rng(1).permutation(n)[:256]
    # reference-style: fanouts listed k-hop..1-hop, with replacement
    npc.set_rng_seed(99)
    sampler = npc.MixedPSNeighborSampler(0, 1, [15, 10, 5], "DP")
    input_nodes, output_nodes, blocks = sampler.sample(None, dev(seeds))
    frontier = seeds
    for hop, (fanout, blk) in enumerate(zip([5, 10, 15], reversed(blocks))):
        nbr, cnt = orc.sample_neighbors(og, frontier, fanout, True, 99, hop)
        uniq, rel = orc.relabel(frontier, nbr)
        keep = rel >= 0
        assert np.array_equal(blk.row.cpu().numpy(), rel[keep])
        assert np.array_equal(blk.col.cpu().numpy(), np.repeat(np.arange(len(frontier)), fanout)[keep])
        assert blk.num_dst == len(frontier) and blk.num_src == len(uniq)
        assert np.array_equal(blk.src_ids.cpu().numpy(), uniq)
        frontier = uniq
    assert np.array_equal(input_nodes.cpu().numpy(), frontier)
    assert np.array_equal(output_nodes.cpu().numpy(), seeds)
    _, x = npc.load_batch(type("A", (), {"system": "DP"})(), (input_nodes, output_nodes, blocks))
    assert np.array_equal(x.cpu().numpy(), feats[frontier])
    host_rows = npc.cpu_load_subtensor(input_nodes.cpu())
    assert host_rows.device.type == "cpu"                      # as the reference's CPU statement returns
    assert np.array_equal(host_rows.numpy(), feats[frontier])
    # a requested node without a row: reported without a wait by default, that is by the next operator call or
    # by check_errors(); by the call itself in "immediate" mode; not at all when switched off
    rows = npc.load_subtensor(torch.tensor([0, n + 5]))
    assert np.array_equal(rows.cpu().numpy()[0], feats[0]) and not rows[1].any()
    with pytest.raises(IndexError, match="earlier call"):
        npc.ops.check_errors()
    npc.ops.check_errors()                                     # reported once
    npc.load_subtensor(torch.tensor([n + 5]))
    torch.cuda.synchronize()
    with pytest.raises(IndexError, match="earlier call"):
        npc.load_subtensor(torch.tensor([3]))                  # the next call reports it
    npc.ops.check_errors()
    npc.ops.set_miss_check("immediate")
    with pytest.raises(IndexError):
        npc.load_subtensor(torch.tensor([0, n + 5]))
    npc.ops.set_miss_check("off")
    npc.load_subtensor(torch.tensor([0, n + 5]))
    npc.ops.check_errors()
    npc.ops.set_miss_check("deferred")
    for _ in range(100):                                       # many calls nobody checks: the queue stays bounded
        npc.load_subtensor(dev(seeds))
    npc.ops.check_errors()
    with pytest.raises(RuntimeError):
        npc.ops.set_miss_check("sometimes")
    with pytest.raises(RuntimeError):
        npc.np_sample_and_shuffle(dev(seeds), 5)
    # the operators are reachable under the reference's names
    u, r = torch.ops.npc.relabel_csc(dev(seeds), dev(seeds[::-1].copy()))
    assert np.array_equal(u.cpu().numpy(), seeds)


def test_operator_relabel_csc_uses_the_rank_table_and_falls_back(orc, capi):
    """relabel_csc on a registered graph: calls above the LDS size go through the graph's rank table, a call
    whose seeds are the unique list of the call before continues that batch, ids the graph does not have make
    the call take the hash table; all give the oracle's answer, as does the operator with the table switched off."""
    import apt_amd as npc
    indptr, indices, feats = _setup(orc, capi, n=50_000, dim=8, seed=6)
    n = len(indptr) - 1
    npc.set_topology(0, 1)
    e = torch.empty(0, dtype=torch.int64)
    npc.mix_cache_graphs(0, e, e, e, torch.from_numpy(indptr), torch.from_numpy(indices))
    rng = np.random.default_rng(4)
    try:
        for ranked in (True, False, True):
            npc.ops.set_ranked_relabel(ranked)
            for chain in range(3):
                frontier = dev(rng.integers(0, n, 3000))
                for f in (4, 6, 5):
                    nbrs = np.where(rng.random(frontier.numel() * f) < 0.05, -1, rng.integers(0, n, frontier.numel() * f))
                    if chain == 2 and f == 6:
                        nbrs[17] = n + 123                           # an id the registered graph does not have
                    want_u, want_r = orc.relabel(frontier.cpu().numpy(), nbrs)
                    u, r = npc.ops.tensor_relabel_csc(frontier, dev(nbrs))
                    assert np.array_equal(u.cpu().numpy(), want_u) and np.array_equal(r.cpu().numpy(), want_r), (ranked, chain, f)
                    frontier = u
    finally:
        npc.ops.set_ranked_relabel(True)


def test_operator_sampling_places_the_bids_of_the_relabel_that_follows(orc, capi):
    """The reference's per-hop pattern through the operators (python/npc/sampler.py:187-203): local_sample_one_layer
    or sample_neighbors, then relabel_csc on the same tensors, the unique list being the next hop's seeds.  The
    sampling operator places the relabel's bids; everything else a caller may do in between -- relabel other
    tensors, sample twice, change the sampled ids in place, pass seeds the graph does not have, switch the rank
    table off -- must give the oracle's answer too."""
    import apt_amd as npc
    indptr, indices, feats = _setup(orc, capi, n=60_000, deg=12, dim=8, seed=16)
    n = len(indptr) - 1
    og = orc.Graph(indptr, indices)
    npc.set_topology(0, 1)
    e = torch.empty(0, dtype=torch.int64)
    npc.mix_cache_graphs(0, e, e, e, torch.from_numpy(indptr), torch.from_numpy(indices))
    rng = np.random.default_rng(9)

    def check_relabel(frontier, nbrs, tag):
        want_u, want_r = orc.relabel(frontier.cpu().numpy(), nbrs.cpu().numpy())
        u, r = npc.ops.tensor_relabel_csc(frontier, nbrs)
        assert np.array_equal(u.cpu().numpy(), want_u), tag
        assert np.array_equal(r.cpu().numpy(), want_r), tag
        return u

    def check_sample(frontier, f, replace, key, hop, tag):
        nbrs, cnt = npc.ops.sample_neighbors(frontier, f, replace, key, hop)
        want_n, want_c = orc.sample_neighbors(og, frontier.cpu().numpy(), f, replace, key, hop)
        assert np.array_equal(nbrs.cpu().numpy(), want_n) and np.array_equal(cnt.cpu().numpy(), want_c), tag
        return nbrs

    try:
        for ranked in (True, False, True):
            npc.ops.set_ranked_relabel(ranked)
            for chain, replace in enumerate((False, True, False, False, False, False)):
                frontier = dev(rng.integers(0, n, 2500))             # repeated seeds happen
                if chain == 5:
                    frontier[7] = n + 5                              # a seed the graph does not have
                for hop, f in enumerate((5, 6, 4)):
                    tag = (ranked, chain, hop)
                    nbrs = check_sample(frontier, f, replace, 700 + chain, hop, tag)
                    if chain == 2 and hop == 1:
                        nbrs = check_sample(frontier, f, replace, 900, hop, tag)        # sampled twice: the first bids are dropped
                    if chain == 3 and hop == 1:
                        other = dev(rng.integers(0, n, 30_000))                         # a relabel of other tensors in between
                        check_relabel(dev(rng.integers(0, n, 4000)), other, tag)
                    if chain == 4 and hop == 2:
                        nbrs[11] = nbrs[12]                                             # changed in place: not what was bid for
                    frontier = check_relabel(frontier, nbrs, tag)
        # the reference's own operator: with replacement, keyed by the call counter
        npc.set_rng_seed(77)
        frontier = dev(rng.permutation(n)[:3000])
        for hop, f in enumerate((5, 5)):
            seeds_out, nbrs = npc.ops.local_sample_one_layer(frontier, f)
            want_n, _ = orc.sample_neighbors(og, frontier.cpu().numpy(), f, True, 77, hop)
            assert np.array_equal(nbrs.cpu().numpy(), want_n)
            frontier = check_relabel(seeds_out, nbrs, ("one_layer", hop))
    finally:
        npc.ops.set_ranked_relabel(True)


def test_operator_sequences_at_random(orc, capi):
    """Random sequences of the sampling and relabel operators on a registered graph -- chains as the reference's
    sampler makes them, chains broken off, relabels of unrelated tensors, repeated sampling, ids changed in place,
    small and large inputs, the rank table switched off and on -- every result against the oracle.  The operators
    keep state between calls (the rank table's batch, bids placed ahead of relabel_csc); no sequence may show it."""
    import apt_amd as npc
    indptr, indices, feats = _setup(orc, capi, n=40_000, deg=10, dim=8, seed=23)
    n = len(indptr) - 1
    og = orc.Graph(indptr, indices)
    npc.set_topology(0, 1)
    e = torch.empty(0, dtype=torch.int64)
    npc.mix_cache_graphs(0, e, e, e, torch.from_numpy(indptr), torch.from_numpy(indices))
    rng = np.random.default_rng(31)
    frontier = nbrs = None
    key = 0
    try:
        for step in range(260):
            what = rng.choice(["seeds", "sample", "sample", "relabel", "relabel", "other", "poke", "toggle"],
                              p=[0.14, 0.2, 0.2, 0.17, 0.17, 0.06, 0.04, 0.02])
            if what == "seeds" or frontier is None:
                frontier = dev(rng.integers(0, n, int(rng.choice([300, 1500, 2600, 4000]))))
                nbrs = None
            elif what == "sample":
                f = int(rng.choice([3, 5, 8]))
                replace = bool(rng.integers(0, 2))
                key += 1
                nbrs, cnt = npc.ops.sample_neighbors(frontier, f, replace, key, step % 5)
                want_n, want_c = orc.sample_neighbors(og, frontier.cpu().numpy(), f, replace, key, step % 5)
                assert np.array_equal(nbrs.cpu().numpy(), want_n) and np.array_equal(cnt.cpu().numpy(), want_c), step
            elif what == "relabel" and nbrs is not None:
                want_u, want_r = orc.relabel(frontier.cpu().numpy(), nbrs.cpu().numpy())
                u, r = npc.ops.tensor_relabel_csc(frontier, nbrs)
                assert np.array_equal(u.cpu().numpy(), want_u) and np.array_equal(r.cpu().numpy(), want_r), step
                if u.numel() < 60_000:                           # the chain goes on from the unique list
                    frontier, nbrs = u, None
                else:
                    frontier = nbrs = None
            elif what == "other":
                a, b = dev(rng.integers(0, n, 2000)), dev(rng.integers(-1, n, 15_000))
                want_u, want_r = orc.relabel(a.cpu().numpy(), b.cpu().numpy())
                u, r = npc.ops.tensor_relabel_csc(a, b)
                assert np.array_equal(u.cpu().numpy(), want_u) and np.array_equal(r.cpu().numpy(), want_r), step
            elif what == "poke" and nbrs is not None:
                nbrs[int(rng.integers(0, nbrs.numel()))] = int(rng.integers(0, n))
            elif what == "toggle":
                npc.ops.set_ranked_relabel(bool(rng.integers(0, 2)))
    finally:
        npc.ops.set_ranked_relabel(True)


def test_cpu_load_subtensor_rejects_ids_without_a_local_row(orc, capi):
    """Ids are checked on the host before anything is enqueued: a node outside the map, or one
    that has no local row (map entry -1, or a cache-only node), raises IndexError."""
    import apt_amd as npc
    n, dim = 1000, 16
    feats = np.random.default_rng(0).standard_normal((600, dim)).astype(np.float32)
    local_idx = torch.arange(0, 600)
    cache = torch.from_numpy(np.random.default_rng(1).standard_normal((50, dim)).astype(np.float32))
    cache_idx = torch.arange(700, 750)
    npc.set_topology(0, 1)
    npc.cache_feats_shared(n, torch.from_numpy(feats), cache, cache_idx, local_idx, 0)
    ok = npc.cpu_load_subtensor(torch.tensor([5, 599, 0, 5]))
    assert np.array_equal(ok.numpy(), feats[[5, 599, 0, 5]])
    assert npc.cpu_load_subtensor(torch.empty(0, dtype=torch.int64)).shape == (0, dim)
    for bad in ([5, 650], [720], [n], [-1], [3, -7, 2]):
        with pytest.raises(IndexError):
            npc.cpu_load_subtensor(torch.tensor(bad))
    torch.cuda.synchronize()                                   # nothing faulted on the device


def test_fused_driver_passes_corrupt_negative_ids_through(orc, capi):
    """An adjacency list that holds negative entries (-2, -3, ... a corrupt file): every negative id
    is padding for the relabel, in the fused driver as in the per-hop one and in the oracle."""
    from apt_amd.pipeline import MiniBatchPipeline
    indptr, indices = small_graph(3000, 12, seed=9)
    indices = indices.copy()
    rng = np.random.default_rng(2)
    hit = rng.permutation(len(indices))[: len(indices) // 10]
    # (the fused driver keeps the 2^32 + 2 most negative values for its own slot states and turns such an id into -1)
    indices[hit] = rng.choice(np.array([-1, -2, -3, -4, -(2 ** 40), np.iinfo(np.int64).min + 2 ** 33]), size=len(hit))
    og = orc.Graph(indptr, indices)
    dg = capi.Graph(dev(indptr), dev(indices))
    hops = [5, 10, 15]
    seeds = rng.permutation(3000)[:256]
    want_in, want_blocks = orc.sample_blocks(og, seeds, hops, False, 31)
    assert any((b["relabeled"] < -1).any() for b in want_blocks)
    for fused in (True, False):
        pipe = MiniBatchPipeline(dg, None, 256, hops, replace=False, fused=fused, gather=False)
        for _ in range(2):
            pipe.run(dev(seeds), 31)
            res = pipe.result()
            assert np.array_equal(res["input_nodes"].cpu().numpy(), want_in)
            assert (res["input_nodes"] >= 0).all()
            for got, want in zip(res["blocks"], want_blocks):
                for k in ("neighbors", "relabeled", "counts", "unique"):
                    assert np.array_equal(got[k].cpu().numpy(), want[k]), (fused, k)


def test_operator_layer_caches_and_buckets(orc, capi):
    import apt_amd as npc
    indptr, indices, feats = _setup(orc, capi, n=6000, dim=24, seed=6)
    n = len(indptr) - 1
    rng = np.random.default_rng(2)
    npc.set_topology(0, 1)
    # graph cache: rows of the 500 highest-degree nodes in a second table
    deg = np.diff(indptr)
    hot = np.argsort(-deg, kind="stable")[:500]
    c_indptr = np.zeros(501, dtype=np.int64)
    c_indptr[1:] = np.cumsum(deg[hot])
    c_indices = np.concatenate([indices[indptr[v]:indptr[v + 1]] for v in hot])
    npc.mix_cache_graphs(500, torch.from_numpy(hot), torch.from_numpy(c_indptr), torch.from_numpy(c_indices),
                         torch.from_numpy(indptr), torch.from_numpy(indices))
    npc.set_rng_seed(5)
    s, nb = npc.local_sample_one_layer(dev(np.arange(n)), 4)
    want, _ = orc.sample_neighbors(orc.Graph(indptr, indices), np.arange(n), 4, True, 5, 0)
    assert np.array_equal(nb.cpu().numpy(), want)
    # feature cache with a column window (the reference's "model parallel" slice)
    local_idx = rng.permutation(n)[:4000]
    cached_idx = np.concatenate([local_idx[:300], np.setdiff1d(np.arange(n), local_idx)[:200]])
    off, Dr = 8, 8
    cache = rng.standard_normal((500, Dr)).astype(np.float32)
    npc.cache_feats_shared(n, torch.from_numpy(feats[:4000]), torch.from_numpy(cache), torch.from_numpy(cached_idx),
                           torch.from_numpy(local_idx), off)
    pos = np.full(n, -1, dtype=np.int64)
    pos[local_idx] = -np.arange(4000) - 2
    pos[cached_idx] = np.arange(500)
    present = np.flatnonzero(pos != -1)
    idx = rng.choice(present, 3000)
    want, miss = orc.gather_rows(orc.FeatStore(feats[:4000], cache, pos, col_offset=off, out_dim=Dr), idx)
    assert miss == 0
    assert np.array_equal(npc.load_subtensor(dev(idx)).cpu().numpy(), want)
    # bucketing: 8 owners on one GPU
    npc.set_topology(rank=2, world_size=8, node_size=8)
    min_vids = np.arange(9) * (n // 8)
    min_vids[-1] = n
    npc.register_min_vids(torch.from_numpy(min_vids), 0)
    ids = rng.integers(0, n, 5000)
    got = npc.cluster_and_permute(dev(ids))
    want = orc.cluster_permute(ids, min_vids, 8, 0, 2, 0, 8)
    for g, w in zip(got, want):
        assert np.array_equal(g.cpu().numpy(), w)
    rwm = np.array([0, 1, 1, 2, 2, 3, 3, 3])
    npc.register_multi_machines_scheme(torch.from_numpy(rwm), torch.arange(4))
    with pytest.raises(RuntimeError):
        npc.shuffle_seeds(dev(ids))                             # world_size 8 needs peers
    got = npc.cluster_reqs(dev(ids))
    want = orc.cluster_reqs(ids, pos, rwm, min_vids, 8, 4)
    assert np.array_equal(got[0].cpu().numpy(), want[0])
    assert np.array_equal(got[1].cpu().numpy(), want[2])
    assert np.array_equal(got[2].cpu().numpy(), want[3])
    # one GPU: shuffle_seeds / feat_shuffle degenerate to local permutes
    npc.set_topology(rank=0, world_size=1)
    npc.register_min_vids(torch.tensor([0, n]), 0)
    recv, perm, recv_off, dev_off = npc.shuffle_seeds(dev(ids))
    assert np.array_equal(recv.cpu().numpy()[perm.cpu().numpy()], ids)
    assert recv_off.tolist() == [5000] and dev_off.tolist() == [5000]
    h = torch.randn(5000, 16, device=DEV)
    fwd = npc.feat_shuffle(h, dev_off, recv_off, perm, 16, 1)
    assert torch.equal(fwd, h[perm])
    bwd = npc.feat_shuffle(fwd, recv_off, dev_off, perm, 16, 0)
    assert torch.equal(bwd, h)                                  # pack undoes unpack (shuffle_seeds' own permutation:
    #                                                             a bijection by construction, taken without a check)
    bwd = npc.feat_shuffle(fwd, recv_off, dev_off, perm.clone(), 16, 0)
    assert torch.equal(bwd, h)                                  # the same values in another tensor: checked, same result
    # the pack direction is index_select_backward (reference src/feat_shuffle.cc:14-16): rows that several
    # entries name add up, rows nobody names are zero
    rep = perm.clone()
    rep[100:300] = perm[0:200]
    rep[4000:4100] = perm[0]
    g = torch.randn(5000, 16, device=DEV)
    got = npc.feat_shuffle(g, recv_off, dev_off, rep, 16, 0)
    want = torch.zeros(5000, 16, device=DEV).index_add_(0, rep, g)
    assert torch.allclose(got, want, rtol=1e-5, atol=1e-4)          # two atomic sums of up to 102 rows, in different orders
    assert bool((got[perm[200:300]] == 0).all()) and bool((got[perm[4000:4100]] == 0).all())
    with pytest.raises(IndexError):
        bad = perm.clone()
        bad[7] = 5000
        npc.feat_shuffle(g, recv_off, dev_off, bad, 16, 0)


def test_partitioned_store_pipeline(orc, capi):
    """One GPU's share: rows [lo, hi) of the graph are here, features of the
    local nodes plus a cache of hot remote nodes; input nodes are bucketed into
    "here" + per-owner request lists and the rows that are here are gathered."""
    from apt_amd.pipeline import MiniBatchPipeline
    indptr, indices, feats = _setup(orc, capi, n=40000, deg=12, dim=64, seed=31)
    n, W = 40000, 8
    lo, hi = 15000, 20000
    p_indptr = indptr[lo:hi + 1] - indptr[lo]
    p_indices = indices[indptr[lo]:indptr[hi]]
    og = orc.Graph(p_indptr, p_indices, row_begin=lo, num_total_nodes=n)
    dg = capi.Graph(dev(p_indptr), dev(p_indices), row_begin=lo, num_total_nodes=n)
    deg = np.diff(indptr)
    remote = np.setdiff1d(np.arange(n), np.arange(lo, hi))
    hot = remote[np.argsort(-deg[remote], kind="stable")[:7000]]            # 20% of the remote nodes
    pos = np.full(n, -1, dtype=np.int64)
    pos[lo:hi] = -np.arange(hi - lo) - 2
    pos[hot] = np.arange(len(hot))
    local_t, cache_t = feats[lo:hi], feats[hot]
    ofs = orc.FeatStore(local_t, cache_t, pos)
    dfs = capi.FeatStore(dev(local_t), dev(cache_t), dev(pos))
    min_vids = np.arange(W + 1) * (n // W)
    rwm = np.arange(W)
    rq = dict(feat_pos_map=dev(pos), remote_worker_map=dev(rwm), min_vids=dev(min_vids), world_size=W,
              num_remote_workers=W)
    hops = [5, 10, 15]
    pipe = MiniBatchPipeline(dg, dfs, 256, hops, replace=False, requests=rq)
    rng = np.random.default_rng(3)
    for batch in range(2):
        seeds = lo + rng.permutation(hi - lo)[:256]
        pipe.run(dev(seeds), 500 + batch)
        res = pipe.result()
        want_in, want_blocks = orc.sample_blocks(og, seeds, hops, False, 500 + batch)
        assert np.array_equal(res["input_nodes"].cpu().numpy(), want_in)
        for got, want in zip(res["blocks"], want_blocks):
            assert np.array_equal(got["relabeled"].cpu().numpy(), want["relabeled"])
        bs, bo, so, pm = orc.cluster_reqs(want_in, pos, rwm, min_vids, W, W)
        assert res["request_sizes"] == bs.tolist()
        assert np.array_equal(res["request_ids"].cpu().numpy(), so)
        assert np.array_equal(res["request_perm"].cpu().numpy(), pm)
        here = so[:bs[0]]
        want_f, _ = orc.gather_rows(ofs, here)
        assert np.array_equal(res["features"].cpu().numpy(), want_f)
        assert bs[1:].sum() > 0 and bs[0] > 0
        # frontier nodes outside the partition have no adjacency here
        outer = want_blocks[0]
        outside = (outer["seeds"] < lo) | (outer["seeds"] >= hi)
        assert outside.any() and np.all(outer["counts"][outside] == 0)


@pytest.mark.parametrize("fuse_mark", [1, 0])
def test_rank_table_epochs_and_refill(orc, capi, fuse_mark):
    """Batches reuse the rank table without clearing it; with a 30-bit id field
    only 3 epochs exist, so the table is refilled every third batch."""
    from apt_amd.pipeline import MiniBatchPipeline
    indptr, indices, _ = _setup(orc, capi, n=20000, deg=10, dim=4, seed=41)
    og = orc.Graph(indptr, indices)
    dg = capi.Graph(dev(indptr), dev(indices))
    hops = [4, 6]
    rng = np.random.default_rng(7)
    capi.set_tuning("minibatch_payload_bits", 30)
    capi.set_tuning("minibatch_fuse_mark", fuse_mark)
    try:
        pipe = MiniBatchPipeline(dg, None, 300, hops, replace=False, gather=False)
        for batch in range(8):
            seeds = rng.integers(0, 20000, size=300)                # overlapping batches, repeated seeds
            pipe.run(dev(seeds), 900 + batch)
            res = pipe.result()
            want_in, want_blocks = orc.sample_blocks(og, seeds, hops, False, 900 + batch)
            assert np.array_equal(res["input_nodes"].cpu().numpy(), want_in), batch
            for got, want in zip(res["blocks"], want_blocks):
                assert np.array_equal(got["relabeled"].cpu().numpy(), want["relabeled"]), batch
    finally:
        capi.set_tuning("minibatch_payload_bits", 0)
        capi.set_tuning("minibatch_fuse_mark", 1)
    # a plan with another id width can take over the same table
    pipe2 = MiniBatchPipeline(dg, None, 64, [3], replace=True, gather=False)
    pipe2.plan.table = pipe.plan.table
    seeds = rng.permutation(20000)[:64]
    pipe2.run(dev(seeds), 5)
    want_in, _ = orc.sample_blocks(og, seeds, [3], True, 5)
    assert np.array_equal(pipe2.result()["input_nodes"].cpu().numpy(), want_in)


def test_batches_in_flight_are_reproducible(orc, capi):
    """Three pipelines on three streams: whatever else is running, a batch with
    the same seeds and rng key gives the same node list and compact ids."""
    from apt_amd import synth
    from apt_amd.pipeline import MiniBatchPipeline
    N = 500_000
    indptr, indices = synth.rmat_csr_gpu(N, 12_000_000, 3, DEV)
    g = capi.Graph(indptr, indices)
    hops = [5, 10, 15]
    pipes = [MiniBatchPipeline(g, None, 1024, hops, gather=False) for _ in range(3)]
    streams = [torch.cuda.Stream() for _ in range(3)]
    gen = torch.Generator(device=DEV)
    gen.manual_seed(9)
    seeds = torch.randperm(N, generator=gen, device=DEV)[:1024].contiguous()
    other = [torch.randperm(N, generator=gen, device=DEV)[:1024].contiguous() for _ in range(4)]
    torch.cuda.synchronize()
    ref = None
    for it in range(12):
        for k in range(3):
            with torch.cuda.stream(streams[k]):
                if k == it % 3:
                    pipes[k].run(seeds, 4242)
                else:
                    pipes[k].run(other[(it + k) % 4], it)
        torch.cuda.synchronize()
        r = pipes[it % 3].result()
        cur = (r["input_nodes"].clone(), [b["relabeled"].clone() for b in r["blocks"]])
        if ref is None:
            ref = cur
            og = orc.Graph(indptr.cpu().numpy(), indices.cpu().numpy())
            want_in, want_blocks = orc.sample_blocks(og, seeds.cpu().numpy(), hops, False, 4242)
            assert np.array_equal(cur[0].cpu().numpy(), want_in)
            for a, b in zip(cur[1], want_blocks):
                assert np.array_equal(a.cpu().numpy(), b["relabeled"])
        else:
            assert torch.equal(cur[0], ref[0]), it
            for a, b in zip(cur[1], ref[1]):
                assert torch.equal(a, b), it


def test_operator_layer_fused_sampler(orc, capi):
    """sample_blocks (all hops in one operator call) through MixedPSNeighborSampler:
    the same batch as the per-hop operators and as the oracle; Block.csc()/csr()."""
    import apt_amd as npc
    indptr, indices, feats = _setup(orc, capi, n=9000, dim=16, seed=8)
    n = len(indptr) - 1
    npc.set_topology(0, 1)
    e = torch.empty(0, dtype=torch.int64)
    npc.mix_cache_graphs(0, e, e, e, torch.from_numpy(indptr), torch.from_numpy(indices))
    og = orc.Graph(indptr, indices)
    rng = np.random.default_rng(4)
    for replace in (False, True):
        fused = npc.MixedPSNeighborSampler(0, 1, [12, 6, 3], "DP", replace=replace, rng_seed=500)
        perhop = npc.MixedPSNeighborSampler(0, 1, [12, 6, 3], "DP", replace=replace, rng_seed=500, fused=False)
        for batch in range(3):                                 # the registry's rank table and workspace are reused
            seeds = rng.permutation(n)[:200]
            a_in, a_out, a_blocks = fused.sample(None, dev(seeds))
            b_in, _, b_blocks = perhop.sample(None, dev(seeds))
            want_in, want_blocks = orc.sample_blocks(og, seeds, [3, 6, 12], replace, 500 + batch)
            assert np.array_equal(a_in.cpu().numpy(), want_in) and torch.equal(a_in, b_in)
            assert torch.equal(a_out, dev(seeds)) and len(a_blocks) == 3
            for a, b, w in zip(a_blocks, b_blocks, want_blocks):
                assert (a.num_src, a.num_dst) == (b.num_src, b.num_dst) == (len(w["unique"]), len(w["seeds"]))
                assert torch.equal(a.row, b.row) and torch.equal(a.col, b.col) and torch.equal(a.src_ids, b.src_ids)
                ref = orc.block_formats(w["relabeled"], a.num_dst, w["fanout"], a.num_src)
                assert np.array_equal(a.row.cpu().numpy(), ref["coo_row"])
                ip, ix, eid = a.csc()
                assert np.array_equal(ip.cpu().numpy(), ref["csc_indptr"]) and np.array_equal(ix.cpu().numpy(), ref["coo_row"])
                assert np.array_equal(eid.cpu().numpy(), np.arange(ref["num_edges"]))
                ip, ix, eid = a.csr()
                assert np.array_equal(ip.cpu().numpy(), ref["csr_indptr"])
                assert np.array_equal(ix.cpu().numpy(), ref["csr_indices"]) and np.array_equal(eid.cpu().numpy(), ref["csr_eids"])
    # a different batch size / fanout list re-plans; a new graph gets a new rank table
    sizes, nodes, hops = npc.ops.sample_blocks(dev(np.arange(50)), [4], False, 9)
    want_in, want_blocks = orc.sample_blocks(og, np.arange(50), [4], False, 9)
    assert sizes[:2] == [50, len(want_in)] and np.array_equal(nodes.cpu().numpy(), want_in)
    assert np.array_equal(hops[0][0].cpu().numpy(), want_blocks[0]["neighbors"])
    assert np.array_equal(hops[0][2].cpu().numpy(), want_blocks[0]["counts"])
    # by default every call returns fresh tensors, as the reference's operators do: three results in a row
    # are three sets of buffers and a held result is never overwritten
    assert npc.ops.block_buffer_ring() == 0
    outs = [npc.ops.sample_blocks(dev(np.arange(50)), [4], False, 10 + k) for k in range(3)]
    keep = (outs[0][1].clone(), outs[0][2][0][1].clone())
    assert len({o[1].data_ptr() for o in outs}) == 3 and len({o[2][0][1].data_ptr() for o in outs}) == 3
    again = npc.ops.sample_blocks(dev(np.arange(50)), [4], False, 10)
    assert torch.equal(outs[0][1], keep[0]) and torch.equal(outs[0][2][0][1], keep[1])   # untouched by later calls
    assert torch.equal(again[1], keep[0]) and torch.equal(again[2][0][1], keep[1])       # same key, same batch
    # opt-in: a ring of two registry-owned sets: a call's tensors stay untouched during the next call and are
    # overwritten by the one after
    npc.ops.set_block_buffer_ring(2)
    assert npc.ops.block_buffer_ring() == 2
    s1, n1, h1 = npc.ops.sample_blocks(dev(np.arange(50)), [4], False, 10)
    s2, n2, h2 = npc.ops.sample_blocks(dev(np.arange(50)), [4], False, 11)
    assert n2.data_ptr() != n1.data_ptr() and torch.equal(n1, keep[0]) and torch.equal(h1[0][1], keep[1])
    s3, n3, h3 = npc.ops.sample_blocks(dev(np.arange(50)), [4], False, 12)
    assert n3.data_ptr() == n1.data_ptr() and h3[0][1].data_ptr() == h1[0][1].data_ptr()
    npc.ops.set_block_buffer_ring(0)
    # the same call with the blocks' COO + CSC emitted before its one wait
    sizes_f, nodes_f, hops_f, fmts = npc.ops.sample_blocks(dev(np.arange(50)), [4], False, 9, formats=True)
    assert sizes_f == sizes and torch.equal(nodes_f, nodes) and torch.equal(hops_f[0][1], hops[0][1])
    alone = npc.ops.block_formats(hops[0][1], 50, 4, nodes.numel(), False)
    assert fmts[0]["num_edges"] == alone["num_edges"] == int((hops[0][1] >= 0).sum())
    for k in ("coo_row", "coo_col", "csc_indptr"):
        assert torch.equal(fmts[0][k], alone[k]), k
    indptr2, indices2, _ = _setup(orc, capi, n=300, dim=4, seed=9)
    npc.mix_cache_graphs(0, e, e, e, torch.from_numpy(indptr2), torch.from_numpy(indices2))
    sizes, nodes, hops = npc.ops.sample_blocks(dev(np.arange(50)), [4], False, 9)
    want_in, _ = orc.sample_blocks(orc.Graph(indptr2, indices2), np.arange(50), [4], False, 9)
    assert np.array_equal(nodes.cpu().numpy(), want_in)


def test_fused_driver_random_configurations(orc, capi):
    """Sixty random plans (1-4 hops, fanouts 1..70 incl. those wider than a wavefront,
    batches 1..3000, with and without replacement, repeated / out-of-range / negative
    seeds, graphs with isolated rows and hubs): fused driver, per-hop driver and oracle
    agree on every array."""
    from apt_amd.pipeline import MiniBatchPipeline
    rng = np.random.default_rng(2024)
    graphs = []
    for seed, (n, deg) in enumerate([(500, 3), (5000, 12), (40000, 25)]):
        indptr, indices = small_graph(n, deg, seed=50 + seed)
        graphs.append((n, orc.Graph(indptr, indices), capi.Graph(dev(indptr), dev(indices))))
    for case in range(60):
        n, og, dg = graphs[case % 3]
        H = int(rng.integers(1, 5))
        hops = [int(rng.choice([1, 2, 3, 5, 8, 15, 16, 17, 33, 64, 70])) for _ in range(H)]
        B = int(rng.choice([1, 2, 63, 64, 65, 300, 1000, 3000]))
        while B * np.prod([1 + f for f in hops]) > 3e6:        # keep the upper-bound buffers small
            hops = hops[:-1] if len(hops) > 1 else [min(hops[0], 15)]
            B = min(B, 300)
        replace = bool(rng.integers(0, 2))
        seeds = rng.integers(0, n, size=B)
        if case % 4 == 1 and B > 2:
            seeds[1] = seeds[0]
            seeds[-1] = -1
        if case % 4 == 2:
            seeds[0] = n + 5                                    # an id the graph does not have
        key = 7000 + case
        for fused in (True, False):
            # the rank table of the fused driver treats an id it cannot hold as padding; the hash table of the
            # per-hop driver keeps it as a node without neighbours
            as_seen = np.where(seeds >= n, -1, seeds) if fused else seeds
            want_in, want_blocks = orc.sample_blocks(og, as_seen, hops, replace, key)
            pipe = MiniBatchPipeline(dg, None, B, hops, replace=replace, gather=False, fused=fused)
            pipe.run(dev(seeds), key)
            res = pipe.result()
            pipe.run(dev(seeds), key)                            # and again on the same buffers and table
            again = pipe.result()
            what = (case, hops, B, replace, fused)
            assert np.array_equal(res["input_nodes"].cpu().numpy(), want_in), what
            assert torch.equal(again["input_nodes"], res["input_nodes"]), what
            assert res["num_edges"] == again["num_edges"] == sum(int(b["counts"].sum()) for b in want_blocks), what
            for got, want in zip(res["blocks"], want_blocks):
                for k in ("neighbors", "relabeled", "counts", "unique"):
                    assert np.array_equal(got[k].cpu().numpy(), want[k]), what + (k,)


def test_deferred_lookup_rides_in_the_gather_or_runs_alone(orc, capi):
    """apt_minibatch_sample_deferred leaves the relabel's last pass to the caller: carried out inside the gather's
    launch, as a launch of its own, or by result() as a last resort, the batch is the one apt_minibatch_sample
    gives.  Many repeated neighbours (a dense little graph), so that plenty of slots lose their race."""
    from apt_amd.pipeline import MiniBatchPipeline
    indptr, indices, feats = _setup(orc, capi, n=3000, deg=40, dim=64, seed=13)
    og = orc.Graph(indptr, indices)
    dg = capi.Graph(dev(indptr), dev(indices))
    fs = capi.FeatStore(dev(feats))
    hops = [5, 10, 15]
    seeds = np.random.default_rng(8).integers(0, 3000, size=700)
    want_in, want_blocks = orc.sample_blocks(og, seeds, hops, False, 3)
    want_f, _ = orc.gather_rows(orc.FeatStore(feats), want_in)
    assert sum(int((b["relabeled"] >= 0).sum()) for b in want_blocks) > 3 * len(want_in)

    def check(res):
        assert np.array_equal(res["input_nodes"].cpu().numpy(), want_in)
        for got, want in zip(res["blocks"], want_blocks):
            for k in ("neighbors", "relabeled", "counts", "unique"):
                assert np.array_equal(got[k].cpu().numpy(), want[k]), k

    pipe = MiniBatchPipeline(dg, fs, 700, hops, replace=False, defer_lookup=True)
    assert pipe.can_defer_lookup and not MiniBatchPipeline(dg, fs, 700, hops).can_defer_lookup   # opt-in
    pipe.sample(dev(seeds), 3, defer_lookup=True)
    assert pipe.plan.pending.open
    torch.cuda.synchronize()
    pending_slots = sum(int((r[: s * f] < -(2 ** 62)).sum()) for r, s, f in
                        zip(pipe.relabeled, pipe.sizes.cpu().tolist(), hops))
    assert pending_slots > 0                                    # the pass really was left out
    pipe.gather()                                               # ... and rides here
    assert not pipe.plan.pending.open
    res = pipe.result()
    check(res)
    assert np.array_equal(res["features"].cpu().numpy(), want_f)
    pipe.sample(dev(seeds), 3, defer_lookup=True)
    pipe.plan.pending.run()                                     # a launch of its own
    check(pipe.result())
    pipe.sample(dev(seeds), 3, defer_lookup=True)
    check(pipe.result())                                        # never gathered: result() carries it out
    pipe.sample(dev(seeds), 3)                                  # not deferred
    assert not pipe.plan.pending.open
    check(pipe.result())
    # a pipeline that has other readers of the compact ids between sampling and gather does not defer
    assert not MiniBatchPipeline(dg, fs, 700, hops, formats="csc", defer_lookup=True).can_defer_lookup
    assert not MiniBatchPipeline(dg, None, 700, hops, gather=False, defer_lookup=True).can_defer_lookup
    # run() the deferred way, eager and as a replayed graph, on rows that are not 16-byte vectors too (the pass
    # then runs on its own inside the same call)
    for store, use_graph in ((fs, False), (fs, True), (capi.FeatStore(dev(feats[:, :63].copy())), False)):
        p2 = MiniBatchPipeline(dg, store, 700, hops, defer_lookup=True, use_graph=use_graph)
        for key in (3, 3):
            p2.run(dev(seeds), key)
            res = p2.result()
            check(res)
            assert res["features"].shape[1] == store.out_dim
