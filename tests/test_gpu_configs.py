"""The benchmark's stated configurations at their stated shapes.

config 1: R-MAT 100 000 nodes / 1.5 M edges (duplicates removed), 100 000 x 128 fp32 features, 1024 seeds
          without repetition, 2 hops with fanouts 5,10 (the reference's order for fan_out 10,5) and 10,5:
          the whole batch against the oracle, bit for bit.
config 3: one GPU's share of the 111 M-node graph: 14 M local rows (a contiguous eighth), their features
          (128 x fp32), a cache of the 20 % hottest remote rows, batch 1024 of local seeds, fanouts 5,10,15;
          rows present here are gathered, the others are bucketed into 8 owner request lists.  The sampled
          blocks and the request lists are compared with the oracle on host copies of the graph and the map;
          the gathered rows with torch's own indexing through the map; plus the properties that hold at any
          size (every id in exactly one bucket, bucket 0 = ids with a row here, misses by owner range, no
          adjacency outside the partition).
config 5: aggregation on the outermost block sampled from that share: mean SpMM at hidden 256 (fp32, bf16)
          and GAT 4 heads x 64 (bf16 in, fp32 accumulate) against the oracle on the copied-back block.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def _close(got, want, rtol):
    return np.max(np.abs(got - want)) <= rtol * (np.abs(want).max() + 1e-30)


@pytest.mark.parametrize("hops", [[5, 10], [10, 5]])
@pytest.mark.parametrize("mode", ["fused", "unfused"])
def test_config1_exact(orc, capi, hops, mode):
    from apt_amd import synth
    from apt_amd.pipeline import MiniBatchPipeline
    N, E, D, B = 100_000, 1_500_000, 128, 1024
    indptr, indices = synth.rmat_csr_numpy(N, E, seed=1)
    assert len(indptr) == N + 1 and len(indices) == E
    feats = np.random.default_rng(2).standard_normal((N, D)).astype(np.float32)
    seeds = np.random.default_rng(3).permutation(N)[:B]
    og, ofs = orc.Graph(indptr, indices), orc.FeatStore(feats)
    pipe = MiniBatchPipeline(capi.Graph(dev(indptr), dev(indices)), capi.FeatStore(dev(feats)), B, hops,
                             replace=False, fused=mode == "fused")
    for key in (11, 12):
        pipe.run(dev(seeds), key)
        res = pipe.result()
        want_in, want_blocks = orc.sample_blocks(og, seeds, hops, False, key)
        assert np.array_equal(res["input_nodes"].cpu().numpy(), want_in)
        assert np.array_equal(want_in[:B], seeds)
        for got, want in zip(res["blocks"], want_blocks):
            for k in ("seeds", "neighbors", "relabeled", "counts", "unique"):
                assert np.array_equal(got[k].cpu().numpy(), want[k]), k
        want_f, miss = orc.gather_rows(ofs, want_in)
        assert miss == 0 and int(pipe.misses.item()) == 0
        assert np.array_equal(res["features"].cpu().numpy(), want_f)
        assert np.array_equal(want_f, feats[want_in])
    # with replacement (the reference's own sampler semantics) on the same inputs
    pipe = MiniBatchPipeline(capi.Graph(dev(indptr), dev(indices)), capi.FeatStore(dev(feats)), B, hops,
                             replace=True, fused=mode == "fused")
    pipe.run(dev(seeds), 13)
    res = pipe.result()
    want_in, want_blocks = orc.sample_blocks(og, seeds, hops, True, 13)
    assert np.array_equal(res["input_nodes"].cpu().numpy(), want_in)
    for got, want in zip(res["blocks"], want_blocks):
        assert np.array_equal(got["relabeled"].cpu().numpy(), want["relabeled"])
    assert np.array_equal(res["features"].cpu().numpy(), feats[want_in])


N3, E3, PARTS, PART, D3, B3 = 111_059_956, 3_200_000_000, 8, 3, 128, 1024
HOPS3 = [5, 10, 15]


@pytest.fixture(scope="module")
def share(capi):
    from apt_amd import synth
    s = synth.partition_share(N3, E3, PARTS, PART, D3, torch.float32, 0.2, 1, DEV)
    yield s
    s.clear()
    torch.cuda.empty_cache()


def _seeds3(share, k):
    gen = torch.Generator(device=DEV)
    gen.manual_seed(40 + k)
    n_local = share["hi"] - share["lo"]
    return (share["lo"] + torch.randperm(n_local, generator=gen, device=DEV)[:B3]).contiguous()


def _pipe3(capi, share, **kw):
    from apt_amd.pipeline import MiniBatchPipeline
    graph = capi.Graph(share["indptr"], share["indices"], row_begin=share["lo"], num_total_nodes=N3)
    store = capi.FeatStore(share["feats"], share["cache"], share["pos_map"])
    requests = dict(feat_pos_map=share["pos_map"], remote_worker_map=share["remote_worker_map"],
                    min_vids=share["min_vids"], world_size=PARTS, num_remote_workers=PARTS)
    return MiniBatchPipeline(graph, store, B3, HOPS3, replace=False, requests=requests, **kw)


def test_config3_share_of_full_graph(orc, capi, share):
    lo, hi = share["lo"], share["hi"]
    n_local, n_cache = hi - lo, share["hot"].numel()
    assert 13_800_000 < n_local < 13_900_000 and share["feats"].shape == (n_local, D3)
    assert n_cache == int((N3 - n_local) * 0.2) and share["cache"].shape == (n_cache, D3)
    assert share["pos_map"].numel() == N3 and share["indices"].numel() > 100_000_000
    assert int(share["indices"].max()) < N3 and int(share["indices"].max()) >= hi     # targets span the global ids
    pos_map, mv, rwm = share["pos_map"], share["min_vids"], share["remote_worker_map"]

    orc.set_threads(16)
    og = orc.Graph(share["indptr"].cpu().numpy(), share["indices"].cpu().numpy(), row_begin=lo, num_total_nodes=N3)
    h_pos, h_mv, h_rw = pos_map.cpu().numpy(), mv.cpu().numpy(), rwm.cpu().numpy()
    pipe = _pipe3(capi, share)
    for k in range(3):
        seeds = _seeds3(share, k)
        pipe.run(seeds, 500 + k)
        res = pipe.result()
        nodes = res["input_nodes"]
        n = nodes.numel()
        # --- sampling + relabel: the oracle on host copies, bit for bit
        want_in, want_blocks = orc.sample_blocks(og, seeds.cpu().numpy(), HOPS3, False, 500 + k)
        assert np.array_equal(nodes.cpu().numpy(), want_in)
        for got, want in zip(res["blocks"], want_blocks):
            for key in ("neighbors", "relabeled", "counts"):
                assert np.array_equal(got[key].cpu().numpy(), want[key]), key
        # --- frontier rows outside the partition have no adjacency here
        left = 0
        for blk in res["blocks"]:
            outside = (blk["seeds"] < lo) | (blk["seeds"] >= hi)
            left += int(outside.sum())
            assert int(blk["counts"][outside].sum()) == 0
            inside = ~outside
            deg = share["indptr"][blk["seeds"][inside] - lo + 1] - share["indptr"][blk["seeds"][inside] - lo]
            assert torch.equal(blk["counts"][inside], torch.clamp(deg, max=blk["fanout"]))
        assert left > 0                                              # the later hops' frontiers do leave the partition
        # --- request lists: the oracle, bit for bit
        bs, bo, so, pm = orc.cluster_reqs(want_in, h_pos, h_rw, h_mv, PARTS, PARTS)
        sizes = res["request_sizes"]
        assert sizes == bs.tolist() and sum(sizes) == n
        ids, perm = res["request_ids"], res["request_perm"]
        assert np.array_equal(ids.cpu().numpy(), so) and np.array_equal(perm.cpu().numpy(), pm)
        assert np.array_equal(pipe.request_offsets.cpu().numpy(), bo)
        # --- and the properties that do not need the oracle
        assert torch.equal(torch.sort(ids).values, torch.sort(nodes).values)          # every id in exactly one bucket
        assert torch.equal(ids[perm], nodes)                                          # permutation[i] = slot of id i
        off = np.concatenate([[0], np.cumsum(sizes)])
        present = pos_map[ids] != -1
        assert bool(present[:sizes[0]].all()) and not bool(present[sizes[0]:].any())  # bucket 0 = rows held here
        assert torch.equal(ids[:sizes[0]], nodes[pos_map[nodes] != -1])               # in input order (stable)
        owner = torch.bucketize(ids, mv[1:PARTS], right=True)
        for b in range(1, PARTS):
            seg = slice(int(off[b]), int(off[b + 1]))
            assert bool((rwm[owner[seg]] == b).all())                                 # misses by owner range
            assert not bool((owner[seg] == PART).any())
            assert torch.equal(ids[seg], nodes[(pos_map[nodes] == -1) & (rwm[owner_of(nodes, mv)] == b)])
        # --- gathered rows of bucket 0 = indexing through the map (the cache wins, local rows otherwise)
        held = ids[:sizes[0]]
        p = pos_map[held]
        want_rows = torch.where((p >= 0)[:, None], share["cache"][p.clamp(min=0)],
                                share["feats"][(-p - 2).clamp(min=0)])
        assert torch.equal(res["features"], want_rows)
        assert int(pipe.misses.item()) == 0
        assert bool((p >= 0).any()) and bool((p < -1).any())                          # both tables were read
    orc.set_threads(1)


def owner_of(ids, min_vids):
    return torch.bucketize(ids, min_vids[1:PARTS], right=True)


def test_config5_aggregation_on_config3_block(orc, capi, share):
    pipe = _pipe3(capi, share)
    pipe.run(_seeds3(share, 7), 700)
    res = pipe.result()
    blk = res["blocks"][0]                                            # outermost hop: fanout 15
    f, n_dst, n_src = blk["fanout"], blk["seeds"].numel(), blk["unique"].numel()
    rel = blk["relabeled"]
    h_rel = rel.cpu().numpy()
    assert f == 15 and n_src == res["input_nodes"].numel() and (h_rel >= 0).sum() == int(blk["counts"].sum())
    rng = np.random.default_rng(4)
    hid = 256
    # GraphSAGE mean over the sampled in-edges: the input is the gathered feature rows' width class (hidden 256)
    x = rng.standard_normal((n_src, hid)).astype(np.float32)
    valid = h_rel.reshape(n_dst, f) >= 0
    col = np.repeat(np.arange(n_dst), f)[valid.reshape(-1)]
    row = h_rel[valid.reshape(-1)]
    cnt = np.maximum(valid.sum(1), 1)[:, None]
    want = orc.spmm_sum(0, row, col, x, n_dst) / cnt
    got = capi.spmm_block(rel, n_dst, f, dev(x), mean=True)
    assert _close(got.cpu().numpy(), want, 1e-5)
    x16 = dev(x).to(torch.bfloat16)
    want16 = orc.spmm_sum(0, row, col, x16.float().cpu().numpy(), n_dst) / cnt
    got16 = capi.spmm_block(rel, n_dst, f, x16, mean=True)
    assert _close(got16.cpu().numpy(), want16, 1e-2)
    # the reference's COO operator on the same block (row = source, col = destination)
    got_coo = capi.spmm_sum(0, dev(row), dev(col), dev(x), n_dst)
    assert _close(got_coo.cpu().numpy(), want * cnt, 1e-5)
    # GAT: 4 heads x 64, bf16 features, fp32 accumulation, weights ~ N(0, 0.02)
    heads, hdim = 4, 64
    ft16 = torch.from_numpy(rng.standard_normal((n_src, heads, hdim)).astype(np.float32)).to(torch.bfloat16)
    ft = ft16.to(torch.float32).numpy()
    al, ar = (rng.standard_normal((2, heads, hdim)) * 0.02).astype(np.float32)
    el = capi.gat_scores(ft16.to(DEV), dev(al))
    er = capi.gat_scores(ft16[:n_dst].contiguous().to(DEV), dev(ar))
    assert _close(el.cpu().numpy(), orc.gat_scores(ft, al), 1e-2)
    assert _close(er.cpu().numpy(), orc.gat_scores(ft[:n_dst], ar), 1e-2)
    want_g, want_a = orc.gat_block(h_rel, n_dst, f, ft, el.cpu().numpy(), er.cpu().numpy(), 0.2, want_attn=True)
    got_g, got_a = capi.gat_block(rel, n_dst, f, ft16.to(DEV), el, er, 0.2, want_attn=True)
    assert _close(got_g.cpu().numpy(), want_g, 1e-2)
    assert np.max(np.abs(got_a.cpu().numpy() - want_a)) <= 1e-2
    # fp32 features: 1e-5
    ft32 = dev(ft)
    el32, er32 = capi.gat_scores(ft32, dev(al)), capi.gat_scores(ft32[:n_dst].contiguous(), dev(ar))
    want32 = orc.gat_block(h_rel, n_dst, f, ft, el32.cpu().numpy(), er32.cpu().numpy(), 0.2)
    assert _close(capi.gat_block(rel, n_dst, f, ft32, el32, er32, 0.2).cpu().numpy(), want32, 1e-5)
    # SDDMM edge scores on the block's COO (u_add_v), fp32
    lhs, rhs = rng.standard_normal((n_src, 64)).astype(np.float32), rng.standard_normal((n_dst, 64)).astype(np.float32)
    assert _close(capi.sddmm(0, dev(row), dev(col), dev(lhs), dev(rhs)).cpu().numpy(),
                  orc.sddmm(0, row, col, lhs, rhs), 1e-5)
