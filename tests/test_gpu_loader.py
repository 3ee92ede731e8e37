"""Epoch loader with mini-batches in flight: every batch equals what one
pipeline builds alone from the same seeds and rng key (bit-exact), an epoch
visits every index once, and buffers are not reused under the consumer."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _setup(capi, n=30000, dim=32):
    import torch

    from apt_amd import synth
    g = capi.Graph(*synth.rmat_csr_gpu(n, 12 * n, seed=9))
    table = synth.random_features(n, dim, torch.float32, seed=4)
    return g, capi.FeatStore(table), table


@pytest.mark.parametrize("in_flight,drop_last,formats,use_graph", [(1, True, False, False), (3, True, "csc", False),
                                                                   (4, False, False, False), (8, False, True, False),
                                                                   (3, False, False, True)])
def test_loader_matches_single_pipeline(capi, in_flight, drop_last, formats, use_graph):
    import torch

    from apt_amd.loader import MiniBatchLoader
    from apt_amd.pipeline import MiniBatchPipeline
    g, store, table = _setup(capi)
    ids = torch.from_numpy(np.random.default_rng(0).choice(30000, 1100, replace=False)).cuda()
    B, hops = 256, [3, 4]
    loader = MiniBatchLoader(g, store, ids, B, hops, in_flight=in_flight, shuffle=True, drop_last=drop_last, seed=5,
                             formats=formats, use_graph=use_graph)
    assert len(loader) == (4 if drop_last else 5)
    ref = {B: MiniBatchPipeline(g, store, B, hops)}
    if not drop_last:
        ref[1100 - 4 * B] = MiniBatchPipeline(g, store, 1100 - 4 * B, hops)
    for epoch in range(2):
        seen, kept = [], []
        for i, batch in enumerate(loader):
            seeds = batch["output_nodes"]
            seen.append(seeds.cpu())
            # consumer work on its own stream that reads the yielded buffers
            kept.append((batch["features"].double().sum(), batch["input_nodes"].sum()))
            pipe = ref[seeds.numel()]
            pipe.run(seeds, (5 * 7919 + epoch) * len(loader) + i)
            want = pipe.result()
            assert torch.equal(batch["input_nodes"], want["input_nodes"])
            assert torch.equal(batch["features"], want["features"])
            assert torch.equal(batch["features"], table[want["input_nodes"]])
            assert batch["num_edges"] == want["num_edges"]
            for b, w in zip(batch["blocks"], want["blocks"]):
                assert torch.equal(b["relabeled"], w["relabeled"]) and torch.equal(b["unique"], w["unique"])
                if formats:
                    assert b["formats"]["num_edges"] == int((w["relabeled"] >= 0).sum())
            kept[-1] += (want["features"].double().sum(), want["input_nodes"].sum())
        assert i + 1 == len(loader)
        got = torch.cat(seen)
        if drop_last:
            assert got.numel() == 4 * B and len(set(got.tolist())) == 4 * B and set(got.tolist()) <= set(ids.tolist())
        else:
            assert sorted(got.tolist()) == sorted(ids.tolist())
        for fs, ns, wf, wn in kept:                      # sums enqueued before the buffers were reused
            assert float(fs) == float(wf) and int(ns) == int(wn)
        if epoch == 0:
            first = got
    assert not torch.equal(first, got)                   # epochs are shuffled differently


def test_loader_without_shuffle_and_early_exit(capi):
    import torch

    from apt_amd.loader import MiniBatchLoader
    g, store, table = _setup(capi)
    ids = torch.arange(100, 100 + 640).cuda()
    loader = MiniBatchLoader(g, store, ids, 128, [5], in_flight=3, shuffle=False)
    for i, batch in enumerate(loader):
        assert torch.equal(batch["output_nodes"], ids[i * 128:(i + 1) * 128])
        assert torch.equal(batch["input_nodes"][:128], batch["output_nodes"])
        if i == 1:
            break                                        # batches 2..4 are in flight; the next epoch starts over
    out = [b["output_nodes"].clone() for b in loader]
    assert torch.equal(torch.cat(out), ids)
    with pytest.raises(ValueError):
        MiniBatchLoader(g, store, ids[:10], 128, [5])


@pytest.mark.parametrize("formats", [False, True])
def test_training_loop_on_the_loader(capi, formats):
    """The loader's batches as Block objects feed apt_amd.layers directly: two SAGE
    layers trained on them learn a label that needs the neighbourhood; with formats=True
    the blocks arrive with COO / CSC / CSR already emitted beside the gather."""
    import torch

    from apt_amd import synth
    from apt_amd.layers import SAGEConv
    from apt_amd.loader import MiniBatchLoader
    from apt_amd.sampler import Block
    n = 4000
    indptr, indices = synth.rmat_csr_numpy(n, n * 10, seed=2)
    g = capi.Graph(torch.from_numpy(indptr).cuda(), torch.from_numpy(indices).cuda())
    gen = torch.Generator().manual_seed(0)
    feats = torch.randn(n, 16, generator=gen)
    deg = np.diff(indptr)
    sums = np.add.reduceat(np.concatenate([feats[:, 0].numpy()[indices], [0.0]]), indptr[:-1]) * (deg > 0)
    labels = torch.from_numpy((sums / np.maximum(deg, 1) > 0).astype(np.int64)).cuda()
    store = capi.FeatStore(feats.cuda())
    torch.manual_seed(0)
    l1, l2 = SAGEConv(16, 32, activation=torch.relu).cuda(), SAGEConv(32, 2).cuda()
    opt = torch.optim.Adam(list(l1.parameters()) + list(l2.parameters()), lr=0.01)
    loader = MiniBatchLoader(g, store, torch.arange(n), 256, [10, 10], in_flight=3, seed=1, formats=formats,
                             as_blocks=True)
    losses = []
    for epoch in range(4):
        for batch in loader:
            blocks = batch["blocks"]
            assert all(isinstance(b, Block) for b in blocks) and blocks[-1].num_dst == 256
            if formats:
                assert blocks[0].formats is not None and "csr_indptr" in blocks[0].formats
            h = l2(blocks[1], l1(blocks[0], batch["features"]))
            loss = torch.nn.functional.cross_entropy(h, labels[batch["output_nodes"]])
            opt.zero_grad()
            loss.backward()
            opt.step()
            losses.append(loss.item())
    assert len(losses) == 4 * 15
    assert np.mean(losses[-10:]) < 0.6 * np.mean(losses[:5]), (losses[:5], losses[-10:])
