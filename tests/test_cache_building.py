"""Cache construction: oracle pins (no GPU) and GPU parity + the property that
caching never changes what sampling and gather return."""
import numpy as np
import pytest

from helpers import small_graph


def test_oracle_count_and_select_closed_forms(orc):
    rng = np.random.default_rng(0)
    ids = np.concatenate([rng.integers(0, 500, 4000), [-1, 500, 777]])
    freq = np.zeros(500, dtype=np.int64)
    orc.count_ids(ids, freq)
    orc.count_ids(ids[:100], freq)
    valid = ids[(ids >= 0) & (ids < 500)]
    v2 = ids[:100]
    assert np.array_equal(freq, np.bincount(valid, minlength=500) + np.bincount(v2, minlength=500))
    indptr, indices = small_graph(1500, 9, seed=4)
    g = orc.Graph(indptr, indices)
    rows = np.concatenate([rng.permutation(1500)[:300], [7, 7, 1499, 0]])
    ip, ix = orc.csr_select_rows(g, rows)
    assert np.array_equal(np.diff(ip), indptr[rows + 1] - indptr[rows])
    assert np.array_equal(ix, np.concatenate([indices[indptr[r]:indptr[r + 1]] for r in rows]))
    # a partition: rows outside have degree 0
    part = orc.Graph(indptr[500:1001] - indptr[500], indices[indptr[500]:indptr[1000]], row_begin=500)
    ip, ix = orc.csr_select_rows(part, np.array([10, 600, 999, 1000]))
    assert np.diff(ip).tolist() == [0, indptr[601] - indptr[600], indptr[1000] - indptr[999], 0]


@pytest.mark.gpu
def test_gpu_count_and_select(orc, capi):
    import torch
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")
    rng = np.random.default_rng(1)
    ids = np.concatenate([rng.integers(0, 5000, 200000), rng.integers(0, 10, 50000), [-1, 5000]])
    freq = torch.zeros(5000, dtype=torch.int64, device="cuda:0")
    capi.count_ids(dev(ids), freq)
    cnt = torch.tensor([1000], dtype=torch.int64, device="cuda:0")
    capi.count_ids(dev(ids), freq, n_dev=cnt)
    want = np.zeros(5000, dtype=np.int64)
    orc.count_ids(ids, want)
    orc.count_ids(ids[:1000], want)
    assert np.array_equal(freq.cpu().numpy(), want)
    from helpers import special_graph
    for indptr, indices in (small_graph(20000, 12, seed=6), special_graph()[:2]):
        n = len(indptr) - 1
        og, dg = orc.Graph(indptr, indices), capi.Graph(dev(indptr), dev(indices))
        rows = np.concatenate([rng.permutation(n)[:min(n, 3000)], [5, 6, 6, 0, n - 1]])
        wp, wx = orc.csr_select_rows(og, rows)
        gp, gx = capi.csr_select_rows(dg, dev(rows))
        assert np.array_equal(gp.cpu().numpy(), wp) and np.array_equal(gx.cpu().numpy(), wx)
    e = capi.csr_select_rows(dg, dev(np.array([], dtype=np.int64)))
    assert e[0].tolist() == [0] and e[1].numel() == 0


def _import_cache():
    """apt_amd refuses to import without its HIP libraries; they are built in-tree
    (no GPU is needed to load them)."""
    from apt_amd import cache
    return cache


def test_policies_closed_forms(tmp_path):
    import torch
    cache = _import_cache()
    g = torch.Generator().manual_seed(0)
    N = 400
    freq = torch.randint(0, 50, (N,), generator=g)
    local = torch.randperm(N, generator=g)[:150]
    # dryrun: hottest local nodes, rows = budget / (dim * 4)
    f, gr = cache.policy_dryrun(freq, local, N, cache_memory=20 * 32 * 4 + 5, input_dim=32)
    order = np.argsort(-freq.numpy(), kind="stable")
    want = [v for v in order if v in set(local.tolist())][:20]
    assert f.tolist() == want and gr.numel() == 0
    f, _ = cache.policy_dryrun(freq, local, N, cache_memory=10 ** 9, input_dim=32)
    assert f.numel() == 150                                   # never more than the local rows
    f, _ = cache.policy_dryrun(freq, local, N, cache_memory=5 * 32 * 4, input_dim=32, base=4)
    assert f.numel() == 20                                    # MP: every rank holds a column slice
    # costmodel: joint id space, the reference's prefix rule
    mem = torch.randint(8, 400, (2 * N,), generator=g)
    ranked = torch.randperm(2 * N, generator=g)
    f, gr = cache.policy_costmodel(ranked, mem, N, cache_memory=9000)
    run = np.cumsum(mem.numpy()[ranked.numpy()])
    first_over = int(np.argmax(run > 9000))
    keep = ranked.numpy()[:max(0, first_over - 1)]
    assert f.tolist() == keep[keep < N].tolist() and gr.tolist() == (keep[keep >= N] - N).tolist()
    assert run[len(keep)] <= 9000 < run[len(keep) + 1]        # one entry short of the budget, as the reference
    f, gr = cache.policy_costmodel(ranked, mem, N, cache_memory=10 ** 9)
    assert f.numel() == 0 and gr.numel() == 0                 # never exceeded -> position 0 -> nothing kept
    # greedy: brute force over m
    fi, gi = torch.randperm(N, generator=g), torch.randperm(N, generator=g)
    for ratio in (0.5, 0.8):
        f, gr = cache.policy_greedy(fi, gi, mem, N, cache_memory=12000, feat_ratio=ratio)
        fm, gm = np.cumsum(mem.numpy()[fi.numpy()]), np.cumsum(mem.numpy()[gi.numpy() + N])
        fits = [m for m in range(N) if fm[int(m * ratio)] + gm[int(m * (1 - ratio))] <= 12000]
        best = max(fits)
        assert fits == list(range(best + 1))                  # monotone, so bisection finds the largest
        assert f.tolist() == fi[:int(best * ratio)].tolist() and gr.tolist() == gi[:int(best * (1 - ratio))].tolist()
    # random
    f, gr = cache.policy_random(local, 0.2, generator=torch.Generator().manual_seed(1))
    assert f.numel() == 30 and len(set(f.tolist())) == 30 and set(f.tolist()) <= set(local.tolist()) and gr.numel() == 0
    # hotness file round trip in the reference's layout
    path = str(tmp_path / "rk#0_epo10.pt")
    cache.save_hotness(path, freq, freq * 2)
    raw = torch.load(path, weights_only=True)
    assert isinstance(raw, list) and len(raw) == 2 and raw[0].dtype == torch.int64
    d, s_ = cache.load_hotness(path)
    assert torch.equal(d, freq) and torch.equal(s_, freq * 2)


@pytest.mark.gpu
def test_dry_run_then_load_partition(orc, capi, tmp_path):
    """Dry run on the pipeline -> hotness file -> policy -> caches built on the GPU
    and registered -> the operators return exactly what they return without caches."""
    import torch

    import apt_amd as npc
    from apt_amd import cache
    from apt_amd.pipeline import MiniBatchPipeline
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")
    indptr, indices = small_graph(30000, 14, seed=8)
    n = 30000
    rng = np.random.default_rng(2)
    feats = rng.standard_normal((n, 48)).astype(np.float32)
    local_ids = np.sort(rng.permutation(n)[:20000])             # rows held here, in this order
    local_feats = feats[local_ids]
    d_indptr, d_indices = dev(indptr), dev(indices)
    graph = capi.Graph(d_indptr, d_indices)
    pipe = MiniBatchPipeline(graph, None, 512, [5, 10], gather=False)
    hot = cache.HotnessCounter(n)
    want_src, want_dst = np.zeros(n, dtype=np.int64), np.zeros(n, dtype=np.int64)
    og = orc.Graph(indptr, indices)
    for b in range(6):
        seeds = rng.permutation(n)[:512]
        pipe.run(dev(seeds), 100 + b)
        hot.add(pipe.nodes, n_dev=pipe.sizes[2:3], output_nodes=dev(seeds))   # no host sync in the loop
        inp, _ = orc.sample_blocks(og, seeds, [5, 10], False, 100 + b)
        orc.count_ids(inp, want_src)
        orc.count_ids(seeds, want_dst)
    assert np.array_equal(hot.src_count.cpu().numpy(), want_src)
    assert np.array_equal(hot.dst_count.cpu().numpy(), want_dst)
    hot.save(str(tmp_path / "rk#0_epo10.pt"))
    freq = cache.load_hotness(str(tmp_path / "rk#0_epo10.pt"), device="cuda:0")[1]
    order = np.argsort(-want_src, kind="stable")
    assert np.array_equal(cache.rank_by_hotness(freq).cpu().numpy(), order)
    # policies: 100 feature rows by the reference's dry-run mode, 1 MiB of adjacency by hotness
    f_ids, none = cache.policy_dryrun(freq, dev(local_ids), n, cache_memory=100 * 48 * 4, input_dim=48)
    is_local = np.zeros(n, dtype=bool)
    is_local[local_ids] = True
    assert none.numel() == 0 and np.array_equal(f_ids.cpu().numpy(), order[is_local[order]][:100])
    g_ids = cache.policy_graph_by_budget(graph, cache.rank_by_hotness(freq), 1 << 20)
    used = np.cumsum((np.diff(indptr)[order] + 1) * 8)
    assert g_ids.numel() == int((used <= (1 << 20)).sum()) and g_ids.numel() > 10
    # build + register
    npc.set_topology(0, 1)
    train_mask = torch.zeros(n, dtype=torch.bool)
    train_mask[::7] = True
    labels = torch.arange(n) % 5
    part = cache.load_partition(0, [0, n], dev(local_ids), dev(local_feats), labels, train_mask, d_indptr, d_indices,
                                f_ids, g_ids, max_cache_feat_nodes=64)
    assert part.num_cached_feat_nodes == 64 and part.num_cached_feat_elements == 64 * 48
    assert part.num_cached_graph_nodes == g_ids.numel()
    assert part.num_cached_graph_elements == int(np.diff(indptr)[g_ids.cpu().numpy()].sum())
    assert np.array_equal(part.train_nid.cpu().numpy(), np.arange(0, n, 7))
    assert np.array_equal(np.nonzero(part.cache_mask.cpu().numpy())[0], np.sort(f_ids.cpu().numpy()[:64]))
    # results through the caches == results without
    npc.set_rng_seed(11)
    ids = dev(rng.integers(0, n, 20000))
    _, nb = npc.local_sample_one_layer(ids, 6)
    want, _ = orc.sample_neighbors(og, ids.cpu().numpy(), 6, True, 11, 0)
    assert np.array_equal(nb.cpu().numpy().reshape(-1, 6), np.asarray(want).reshape(-1, 6))
    have = dev(local_ids[rng.integers(0, len(local_ids), 20000)])
    x = npc.load_subtensor(have)
    assert np.array_equal(x.cpu().numpy(), feats[have.cpu().numpy()])
    with pytest.raises(IndexError):
        cache.build_feature_cache(dev(local_feats), dev(local_ids), n, dev(np.setdiff1d(np.arange(n), local_ids)[:5]))
    # MP: a column slice of the cached rows
    sl = cache.build_feature_cache(dev(local_feats), dev(local_ids), n, f_ids, 16, 40)
    assert np.array_equal(sl.cpu().numpy(), feats[f_ids.cpu().numpy(), 16:40])
