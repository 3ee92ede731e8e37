"""Strategy cost model (reference python/npc/cost_model/estimator.py) and the
all-strategies dry run (python/npc/sampler.py:367-600).  The arithmetic is checked
against numbers worked out by hand; the dry run's sizes and node sets against
numpy closed forms of the samples it drew."""
import numpy as np
import pytest


def test_volume_and_time_arithmetic():
    import torch

    from apt_amd import cost_model as cm
    # 6 accesses in all, cache of the 2 hottest nodes of the ranking keeps 3 + 2 -> 1 miss, x dim 10
    freq = torch.tensor([3, 0, 2, 1])
    assert int(cm.get_cache_miss(freq, 2, 10)) == 10
    # ranked by another frequency: its two hottest are nodes 1 and 3 -> misses 3 + 2
    assert int(cm.get_cache_miss(freq, 2, 10, made_seeds_freq=torch.tensor([0, 9, 1, 5]))) == 50
    assert int(cm.get_cache_miss(freq, 99, 10)) == 0
    # 1 MiB worth of fp32 elements at BW_PCIE MB/s
    assert cm.cachemiss_vol_to_time(262144) == pytest.approx(1.0 / cm.BW_PCIE)
    assert cm.cpu_cachemiss_vol_to_time(262144) == pytest.approx(1.0 / cm.BW_PURE_NETWORK)
    assert cm.reshuffle_vol_to_time(262144) == pytest.approx(1.0 / cm.BW_NETWORK)
    t = cm.get_featload_time(freq, 1, 8, gpu_sorted_idx=torch.tensor([2, 0, 1, 3]))   # caches node 2 only: 4 misses
    assert float(t) == pytest.approx(4 * 8 * 4 / (1024 * 1024 * cm.BW_PCIE))
    assert cm.get_reshuffle_dim("SAGE", 32, 4) == 32 and cm.get_reshuffle_dim("GAT", 32, 4) == 128
    # inclusive offsets of bucket sizes [4, 1, 7] / [2, 5, 3]; rank 1 keeps its own bucket
    assert cm.get_np_reshuffle_vol(1, 3, 16, [4, 5, 12], [2, 7, 10]) == 2 * 16 * ((4 + 7) + (2 + 3))
    assert cm.get_np_reshuffle_vol(0, 3, 16, [4, 5, 12], [2, 7, 10]) == 2 * 16 * ((1 + 7) + (5 + 3))
    # SP, per peer (ids, virtual nodes): only the virtual nodes of the other ranks count
    assert cm.get_sp_reshuffle_vol(0, 2, 8, [10, 3, 20, 5], [10, 3, 30, 7]) == 2 * 8 * (5 + 7)
    # with destinations, per peer (dst, ids, virtual nodes): dst and virtual nodes
    assert cm.get_sp_reshuffle_vol(1, 2, 8, [2, 10, 3, 4, 20, 5], [6, 10, 7, 4, 20, 5], "SAGE", True) == 2 * 8 * (2 + 3 + 6 + 7)
    assert cm.get_sp_reshuffle_vol(1, 3, 16, [4, 5, 12], [2, 7, 10], "GAT") == cm.get_np_reshuffle_vol(1, 3, 16, [4, 5, 12], [2, 7, 10])
    assert cm.get_mp_reshuffle_vol(4, 8, 100, [100, 90, 80, 70]) == 2 * 8 * (100 * 2 + 340)
    assert cm.get_dp_reshuffle_vol() == 0
    assert cm.pick_strategy({"DP": [1, 2, 0], "NP": [1, 1, 0.5], "SP": [3, 0, 0], "MP": [0.5, 1, 1]}) == "NP"
    assert cm.pick_strategy({"DP": [1], "NP": [1], "SP": [1], "MP": [1]}) == "DP"
    assert cm.SYSTEM_NAMES["SP"] == "SNP"


def _owner(v, min_vids):
    return np.searchsorted(min_vids[1:-1], v, side="right")


def _first_unique(x):
    _, i = np.unique(x, return_index=True)
    return x[np.sort(i)]


@pytest.mark.gpu
@pytest.mark.parametrize("world,model,with_dst", [(1, "SAGE", False), (4, "SAGE", False), (4, "GCN", False),
                                                  (3, "SAGE", True), (4, "GAT", False), (2, "GAT", True)])
def test_gpu_dry_run_sizes_and_node_sets(capi, world, model, with_dst):
    import torch

    from apt_amd import cost_model as cm
    from apt_amd import synth
    n, fanouts = 20000, [4, 3]                       # walked in reverse: seeds use 3, last hop 4
    g = capi.Graph(*synth.rmat_csr_gpu(n, 15 * n, seed=5))
    min_vids = np.linspace(0, n, world + 1).astype(np.int64)
    rng = np.random.default_rng(world)
    seeds = [torch.from_numpy(rng.choice(n, 200, replace=False)).cuda() for _ in range(world)]
    run = cm.AllPSDryRun(g, world, fanouts, torch.from_numpy(min_vids), model=model, shuffle_with_dst=with_dst,
                         rng_seed=11, keep_samples=True)
    res = run.sample(seeds)
    assert len(res) == world
    fanout = fanouts[0]
    fr = [r.frontier.cpu().numpy() for r in res]
    nb = [r.neighbors.cpu().numpy() for r in res]
    for r in range(world):
        assert np.array_equal(fr[r][:200], seeds[r].cpu().numpy())
        ok = nb[r] >= 0
        # DP: first-occurrence unique of (frontier, neighbours)
        dp = _first_unique(np.concatenate([fr[r], nb[r][ok]]))
        assert np.array_equal(res[r].dp_seeds.cpu().numpy(), dp)
        # NP: bucket sizes by owner, the owner's receive sizes by sender
        send = np.bincount(_owner(fr[r], min_vids), minlength=world)
        assert res[r].np_send_offset == np.cumsum(send).tolist()
        recv = [int((_owner(fr[q], min_vids) == r).sum()) for q in range(world)]
        assert res[r].np_recv_offset == np.cumsum(recv).tolist()
        mine = np.unique(np.concatenate([fr[q][_owner(fr[q], min_vids) == r] for q in range(world)]))
        got = res[r].np_seeds.cpu().numpy()
        assert np.array_equal(got[:len(mine)], mine)                 # owners sample each of their nodes once
        assert len(np.unique(got)) == len(got)
        # MP: everyone's input nodes, sizes of the seeds (frontier) or of the unique lists
        assert np.array_equal(res[r].mp_seeds.cpu().numpy(), np.concatenate([x.dp_seeds.cpu().numpy() for x in res]))
        sizes = [len(x.dp_seeds) for x in res] if model == "GAT" else [len(f) for f in fr]
        assert res[r].mp_send_size == sizes[r] and res[r].mp_recv_size == sizes

    # SP
    for r in range(world):
        ok = nb[r] >= 0
        src = nb[r][ok]
        dst_idx = (np.arange(len(nb[r])) // fanout)[ok]
        own = _owner(src, min_vids)
        if model == "GAT":
            ids = np.unique(src)
            if with_dst:
                ids = np.concatenate([fr[r], ids])
            send = np.bincount(_owner(ids, min_vids), minlength=world)
            assert res[r].sp_send_sizes == np.cumsum(send).tolist()
            continue
        per = 3 if with_dst else 2
        for q in range(world):
            pairs = {(int(o), int(d)) for o, d in zip(own, dst_idx) if o == q}
            got = res[r].sp_send_sizes[per * q:per * (q + 1)]
            want = [int((own == q).sum()), len(pairs)]
            if with_dst:
                want = [int((_owner(fr[r], min_vids) == q).sum())] + want
            assert got == want, (r, q, got, want)
    for q in range(world):
        got = res[q].sp_seeds.cpu().numpy()
        srcs = [nb[r][nb[r] >= 0] for r in range(world)]
        if model == "GAT":
            uniq = [np.unique(s) for s in srcs]
            if with_dst:
                uniq = [np.concatenate([fr[r], uniq[r]]) for r in range(world)]
            recv = np.concatenate([u[_owner(u, min_vids) == q] for u in uniq])
            want = recv if with_dst else np.concatenate([fr[q], recv])
            assert np.array_equal(np.sort(got), np.sort(want))
            continue
        per = 3 if with_dst else 2
        assert res[q].sp_recv_sizes == [res[r].sp_send_sizes[per * q + i] for r in range(world) for i in range(per)]
        mine = np.unique(np.concatenate([s[_owner(s, min_vids) == q] for s in srcs]))
        if with_dst:
            dsts = np.concatenate([fr[r][_owner(fr[r], min_vids) == q] for r in range(world)])
            assert np.array_equal(np.sort(got[:len(dsts)]), np.sort(dsts)) and np.array_equal(got[len(dsts):], mine)
        elif model == "GCN":
            assert np.array_equal(got, mine)
        else:
            assert np.array_equal(got, np.concatenate([fr[q], mine]))
    if world == 1:      # nothing leaves the rank: every strategy loads DP's nodes and reshuffles nothing
        r0 = res[0]
        assert set(r0.np_seeds.tolist()) == set(r0.dp_seeds.tolist())
        if model != "GCN":
            assert set(r0.sp_seeds.tolist()) == set(r0.dp_seeds.tolist())
        assert cm.get_np_reshuffle_vol(0, 1, 8, r0.np_send_offset, r0.np_recv_offset) == 0
        assert cm.get_sp_reshuffle_vol(0, 1, 8, r0.sp_send_sizes, r0.sp_recv_sizes) == 0


@pytest.mark.gpu
def test_gpu_estimate_prefers_cheaper_strategy(capi):
    """With one rank nothing is exchanged; with a cache that holds every node no
    feature is loaded: the estimate is then the sampling time alone.  With several
    ranks MP's volume is the closed form of the frontier sizes."""
    import torch

    from apt_amd import cost_model as cm
    from apt_amd import synth
    n, world = 20000, 4
    g = capi.Graph(*synth.rmat_csr_gpu(n, 15 * n, seed=6))
    min_vids = torch.from_numpy(np.linspace(0, n, world + 1).astype(np.int64))
    rng = np.random.default_rng(2)
    batches = [[torch.from_numpy(rng.choice(n, 128, replace=False)).cuda() for _ in range(world)] for _ in range(3)]
    run = cm.AllPSDryRun(g, world, [5, 5], min_vids, rng_seed=3)
    est = cm.estimate(run, batches, rank=1, input_dim=64, num_hidden=32, cache_memory=n * 64 * 4)
    assert set(est.costs) == set(cm.STRATEGIES) and est.best in cm.STRATEGIES
    for s in cm.STRATEGIES:
        sampling, load, reshuffle = est.costs[s]
        assert sampling > 0 and load == 0
    assert est.costs["DP"][2] == 0 and est.costs["MP"][2] > 0
    assert est.best_system == cm.SYSTEM_NAMES[est.best]
    # no cache: DP loads every input node's whole row, MP a quarter of the row of four ranks' input nodes
    est0 = cm.estimate(run, batches, rank=1, input_dim=64, num_hidden=32, cache_memory=0)
    assert est0.costs["DP"][1] > 0 and est0.costs["MP"][1] > 0
