"""Layers over sampled blocks: gradients against torch's own dense arithmetic, a
GAT layer against its textbook statement, and a short training run."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _setup_graph(n=6000, deg=8, seed=0):
    from helpers import small_graph
    import apt_amd as npc
    indptr, indices = small_graph(n, deg, seed=seed)
    npc.set_topology(0, 1)
    e = torch.empty(0, dtype=torch.int64)
    npc.mix_cache_graphs(0, e, e, e, torch.from_numpy(indptr), torch.from_numpy(indices))
    return indptr, indices


def test_block_aggregate_gradients():
    import apt_amd as npc
    from apt_amd.layers import BlockAggregate
    _setup_graph()
    sampler = npc.MixedPSNeighborSampler(0, 1, [7, 4], "DP", replace=False, rng_seed=3)
    seeds = torch.from_numpy(np.random.default_rng(0).permutation(6000)[:300]).to(DEV)
    _, _, blocks = sampler.sample(None, seeds)
    for blk in blocks:
        for mean in (False, True):
            X = torch.randn(blk.num_src, 24, device=DEV, requires_grad=True)
            out = BlockAggregate.apply(blk, X, mean)
            w = torch.randn_like(out)
            (out * w).sum().backward()
            X2 = X.detach().clone().requires_grad_(True)
            ref = torch.zeros(blk.num_dst, 24, device=DEV).index_add(0, blk.col, X2[blk.row])
            if mean:
                cnt = torch.bincount(blk.col, minlength=blk.num_dst).clamp(min=1)
                ref = ref / cnt[:, None]
            (ref * w).sum().backward()
            assert torch.allclose(out, ref, rtol=1e-5, atol=1e-5)
            assert torch.allclose(X.grad, X2.grad, rtol=1e-5, atol=1e-5)
            # the forward is reproducible bit for bit; so is the backward except for source rows whose edges
            # span more than two wavefront ranges (hubs), which are added atomically
            X3 = X.detach().clone().requires_grad_(True)
            out3 = BlockAggregate.apply(blk, X3, mean)
            (out3 * w).sum().backward()
            assert torch.equal(out3, out) and torch.allclose(X3.grad, X.grad, rtol=1e-6, atol=1e-6)
    # a bf16 model: sums are fp32 inside the kernels, results come back in the input's dtype
    X16 = torch.randn(blocks[0].num_src, 32, device=DEV).to(torch.bfloat16).requires_grad_(True)
    out16 = BlockAggregate.apply(blocks[0], X16, True)
    assert out16.dtype == torch.bfloat16
    out16.float().sum().backward()
    assert X16.grad.dtype == torch.bfloat16
    ref16 = BlockAggregate.apply(blocks[0], X16.detach().float(), True)
    assert torch.allclose(out16.float(), ref16, rtol=1e-2, atol=1e-2)


def test_graphconv_matches_dense_statement():
    import apt_amd as npc
    from apt_amd.layers import GraphConv
    _setup_graph(seed=4)
    sampler = npc.MixedPSNeighborSampler(0, 1, [5], "DP", replace=True, rng_seed=6)
    seeds = torch.from_numpy(np.random.default_rng(2).permutation(6000)[:150]).to(DEV)
    _, _, (blk,) = sampler.sample(None, seeds)
    for norm, scale in (("both", 1 / 5.0), ("right", 1 / 5.0), ("left", 1 / 5.0), ("none", 1.0)):
        layer = GraphConv(12, 7, norm=norm).to(DEV)
        feat = torch.randn(blk.num_src, 12, device=DEV, requires_grad=True)
        got = layer(blk, feat)
        h = feat @ layer.weight
        want = torch.zeros(blk.num_dst, 7, device=DEV).index_add(0, blk.col, h[blk.row]) * scale + layer.bias
        assert torch.allclose(got, want, rtol=1e-5, atol=1e-5), norm
        g1, = torch.autograd.grad(got.sum(), feat, retain_graph=True)
        g2, = torch.autograd.grad(want.sum(), feat)
        assert torch.allclose(g1, g2, rtol=1e-5, atol=1e-5), norm


def test_gat_layer_matches_dense_statement():
    import apt_amd as npc
    from apt_amd.layers import GATConv
    _setup_graph(seed=1)
    sampler = npc.MixedPSNeighborSampler(0, 1, [6], "DP", replace=False, rng_seed=5)
    seeds = torch.from_numpy(np.random.default_rng(1).permutation(6000)[:200]).to(DEV)
    _, _, (blk,) = sampler.sample(None, seeds)
    layer = GATConv(16, 8, 3).to(DEV)
    feat = torch.randn(blk.num_src, 16, device=DEV)
    with torch.no_grad():
        got = layer(blk, feat)
        ft = layer.fc(feat).view(-1, 3, 8)
        el, er = (ft * layer.attn_l).sum(-1), (ft[:blk.num_dst] * layer.attn_r).sum(-1)
        e = torch.nn.functional.leaky_relu(el[blk.row] + er[blk.col], 0.2)            # [E, H]
        top = torch.full((blk.num_dst, 3), -1e30, device=DEV).scatter_reduce(0, blk.col[:, None].expand(-1, 3), e, "amax")
        w = torch.exp(e - top[blk.col])
        den = torch.zeros(blk.num_dst, 3, device=DEV).index_add(0, blk.col, w)
        a = w / den[blk.col]
        want = torch.zeros(blk.num_dst, 3, 8, device=DEV).index_add(0, blk.col, a[:, :, None] * ft[blk.row])
        want = want + layer.bias.view(1, 3, 8)
    assert torch.allclose(got, want, rtol=1e-4, atol=1e-5)


def _gat_dense(layer, blk, feat):
    """The layer's textbook statement in plain torch (autograd gives the reference gradients)."""
    H, D = layer.num_heads, layer.out_feats
    ft = layer.fc(feat).view(-1, H, D)
    el, er = (ft * layer.attn_l).sum(-1), (ft[:blk.num_dst] * layer.attn_r).sum(-1)
    e = torch.nn.functional.leaky_relu(el[blk.row] + er[blk.col], layer.negative_slope)
    top = torch.full((blk.num_dst, H), -1e30, device=DEV).scatter_reduce(0, blk.col[:, None].expand(-1, H), e.detach(), "amax")
    w = torch.exp(e - top[blk.col])
    den = torch.zeros(blk.num_dst, H, device=DEV).index_add(0, blk.col, w)
    a = w / den[blk.col]
    out = torch.zeros(blk.num_dst, H, D, device=DEV).index_add(0, blk.col, a[:, :, None] * ft[blk.row])
    return out + layer.bias.view(1, H, D)


@pytest.mark.parametrize("heads,dim,fanout", [(3, 8, 9), (4, 64, 9), (1, 5, 9), (2, 100, 9),      # lane-group kernels
                                              (4, 64, 16), (8, 8, 8), (1, 256, 15), (2, 16, 3)])    # wavefront per destination
def test_gat_layer_gradients(heads, dim, fanout):
    import apt_amd as npc
    from apt_amd.layers import GATConv
    _setup_graph(seed=5)
    sampler = npc.MixedPSNeighborSampler(0, 1, [fanout], "DP", replace=False, rng_seed=8)
    seeds = torch.from_numpy(np.random.default_rng(3).permutation(6000)[:300]).to(DEV)
    _, _, (blk,) = sampler.sample(None, seeds)
    torch.manual_seed(1)
    layer = GATConv(20, dim, heads).to(DEV)
    feat = torch.randn(blk.num_src, 20, device=DEV, requires_grad=True)
    w = torch.randn(blk.num_dst, heads, dim, device=DEV)
    got = layer(blk, feat)
    params = [feat, layer.fc.weight, layer.attn_l, layer.attn_r]
    g_got = torch.autograd.grad((got * w).sum(), params)
    want = _gat_dense(layer, blk, feat)
    g_want = torch.autograd.grad((want * w).sum(), params)
    assert torch.allclose(got, want, rtol=1e-4, atol=1e-5)
    for a, b, name in zip(g_got, g_want, ("feat", "fc", "attn_l", "attn_r")):
        scale = b.abs().max().item() + 1e-12
        assert (a - b).abs().max().item() <= 2e-4 * scale, (name, (a - b).abs().max().item(), scale)


@pytest.mark.parametrize("heads,dim", [(4, 64), (2, 16), (3, 24), (1, 40), (8, 8), (1, 256)])
def test_gat_backward_bf16_matches_fp32_on_rounded_inputs(capi, heads, dim):
    """bf16 features take other kernel variants (8 per lane); on the same (rounded)
    values they must give what the fp32 variants give."""
    rng = np.random.default_rng(heads * 100 + dim)
    n_dst, fanout, n_src = 2000, 11, 9000
    nbr = rng.integers(0, n_src, size=(n_dst, fanout)).astype(np.int64)
    nbr[rng.random(nbr.shape) < 0.2] = -1
    nbr = torch.from_numpy(nbr.reshape(-1)).to(DEV)
    ft16 = torch.randn(n_src, heads, dim, device=DEV).to(torch.bfloat16)
    ft32 = ft16.float()
    el, er = torch.randn(n_src, heads, device=DEV), torch.randn(n_dst, heads, device=DEV)
    d_out = torch.randn(n_dst, heads, dim, device=DEV)
    fmt = capi.block_formats(nbr, n_dst, fanout, n_src, want_csr=False)
    outs = []
    for ft in (ft32, ft16):
        _, attn = capi.gat_block(nbr, n_dst, fanout, ft, el, er, 0.2, want_attn=True)
        outs.append(capi.gat_block_backward(nbr, n_dst, fanout, ft, el, er, 0.2, attn, d_out, fmt["csc_indptr"],
                                            fmt["num_edges"]))
    for a, b in zip(*outs):
        assert torch.allclose(a, b, rtol=1e-4, atol=1e-5)


def test_sage_trains_on_sampled_batches():
    """Two SAGE layers on sampled blocks + gathered features learn a label that
    depends on the neighbourhood: the loss falls well below its start."""
    import apt_amd as npc
    from apt_amd.layers import SAGEConv
    indptr, indices = _setup_graph(n=4000, deg=10, seed=2)
    n = 4000
    g = torch.Generator().manual_seed(0)
    feats = torch.randn(n, 16, generator=g)
    # label: sign of the mean of feature 0 over the in-neighbours (needs aggregation to predict)
    nb_mean = np.array([feats[indices[indptr[v]:indptr[v + 1]], 0].mean().item() if indptr[v + 1] > indptr[v] else 0.0
                        for v in range(n)])
    labels = torch.from_numpy((nb_mean > 0).astype(np.int64)).to(DEV)
    npc.cache_feats_shared(n, feats, torch.empty(0, 16), torch.empty(0, dtype=torch.int64), torch.arange(n), 0)
    torch.manual_seed(0)
    l1, l2 = SAGEConv(16, 32, activation=torch.relu).to(DEV), SAGEConv(32, 2).to(DEV)
    opt = torch.optim.Adam(list(l1.parameters()) + list(l2.parameters()), lr=0.01)
    sampler = npc.MixedPSNeighborSampler(0, 1, [10, 10], "DP", replace=False, rng_seed=11)
    rng = np.random.default_rng(3)
    losses = []
    for step in range(60):
        seeds = torch.from_numpy(rng.permutation(n)[:256]).to(DEV)
        input_nodes, output_nodes, blocks = sampler.sample(None, seeds)
        x = npc.load_subtensor(input_nodes)
        h = l2(blocks[1], l1(blocks[0], x))
        loss = torch.nn.functional.cross_entropy(h, labels[output_nodes])
        opt.zero_grad()
        loss.backward()
        opt.step()
        losses.append(loss.item())
    assert np.mean(losses[-10:]) < 0.6 * np.mean(losses[:5]), (losses[:5], losses[-10:])
