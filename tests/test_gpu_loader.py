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


def test_loader_c_and_python_drivers_agree(capi):
    """The C library's epoch thread and the Python enqueue path build the same batches; the C path is what a
    loader without formats uses by default."""
    import torch

    from apt_amd.loader import MiniBatchLoader
    g, store, table = _setup(capi)
    ids = torch.arange(3000, 3000 + 2100).cuda()
    kw = dict(in_flight=3, shuffle=True, drop_last=False, seed=11)
    a = MiniBatchLoader(g, store, ids, 200, [4, 3, 2], driver="c", **kw)
    b = MiniBatchLoader(g, store, ids, 200, [4, 3, 2], driver="python", **kw)
    assert a._use_c and not b._use_c and MiniBatchLoader(g, store, ids, 200, [4], **kw)._use_c
    assert MiniBatchLoader(g, store, ids, 200, [4], formats=True, **kw)._use_c
    with pytest.raises(ValueError):
        MiniBatchLoader(g, store, ids, 200, [4], driver="c", use_graph=True)
    # the caller's own streams (one per batch in flight, never the default stream)
    mine = [torch.cuda.Stream() for _ in range(3)]
    a = MiniBatchLoader(g, store, ids, 200, [4, 3, 2], driver="c", streams=mine, **kw)
    assert [st.cuda_stream for st in a.streams] == [st.cuda_stream for st in mine]
    with pytest.raises(ValueError):
        MiniBatchLoader(g, store, ids, 200, [4], streams=mine[:2], **kw)
    with pytest.raises(ValueError):
        MiniBatchLoader(g, store, ids, 200, [4], streams=[torch.cuda.default_stream()] * 3, **kw)
    for epoch in range(2):
        n = 0
        for x, y in zip(a, b):
            assert torch.equal(x["output_nodes"], y["output_nodes"]) and x["sizes"] == y["sizes"]
            assert torch.equal(x["input_nodes"], y["input_nodes"]) and torch.equal(x["features"], y["features"])
            assert x["num_edges"] == y["num_edges"]
            for p, q in zip(x["blocks"], y["blocks"]):
                for k in ("seeds", "neighbors", "relabeled", "counts", "unique"):
                    assert torch.equal(p[k], q[k]), k
            n += 1
        assert n == 11
    # block formats through either driver: COO + CSC + CSR, and COO + CSC only
    for formats in (True, "csc", "inner"):
        a = MiniBatchLoader(g, store, ids, 200, [4, 3, 2], driver="c", formats=formats, **kw)
        b = MiniBatchLoader(g, store, ids, 200, [4, 3, 2], driver="python", formats=formats, **kw)
        n = 0
        for x, y in zip(a, b):
            assert torch.equal(x["input_nodes"], y["input_nodes"]) and torch.equal(x["features"], y["features"])
            for p, q in zip(x["blocks"], y["blocks"]):
                assert torch.equal(p["relabeled"], q["relabeled"])
                fp, fq = p["formats"], q["formats"]
                assert fp["num_edges"] == fq["num_edges"] == int((p["relabeled"] >= 0).sum())
                outermost = p is x["blocks"][0]
                assert sorted(fp) == sorted(fq)
                assert ("csr_indptr" in fp) == (formats is True or (formats == "inner" and not outermost))
                for k in fp:
                    if k != "num_edges":
                        assert torch.equal(fp[k], fq[k]), (formats, k)
            n += 1
        assert n == 11


def test_loader_with_partitioned_store(capi):
    """A partitioned feature store through the loader: request lists and the rows held here are what a lone
    pipeline produces for the same seeds and key."""
    import torch

    from apt_amd import synth
    from apt_amd.loader import MiniBatchLoader
    from apt_amd.pipeline import MiniBatchPipeline
    n, lo, hi, dim, P = 30000, 10000, 20000, 16, 4
    indptr, indices = synth.rmat_csr_gpu(n, 12 * n, seed=9)
    g = capi.Graph((indptr[lo:hi + 1] - indptr[lo]).contiguous(), indices[int(indptr[lo]):int(indptr[hi])].clone(),
                   row_begin=lo, num_total_nodes=n)
    local = synth.random_features(hi - lo, dim, torch.float32, seed=4)
    hot = torch.cat([torch.arange(0, 3000), torch.arange(25000, 26000)]).cuda()
    cache = synth.random_features(hot.numel(), dim, torch.float32, seed=5)
    pos = torch.full((n,), -1, dtype=torch.int64, device="cuda")
    pos[lo:hi] = -torch.arange(hi - lo, device="cuda") - 2
    pos[hot] = torch.arange(hot.numel(), device="cuda")
    store = capi.FeatStore(local, cache, pos)
    rq = dict(feat_pos_map=pos, remote_worker_map=torch.tensor([1, 0, 2, 3], device="cuda"),
              min_vids=torch.tensor([0, 10000, 20000, 25000, 30000], device="cuda"), world_size=P, num_remote_workers=P)
    ids = torch.arange(lo, lo + 1280).cuda()
    for driver, formats in (("c", False), ("python", False), ("c", True)):
        lone = MiniBatchPipeline(g, store, 128, [4, 4], requests=rq, formats=formats)
        loader = MiniBatchLoader(g, store, ids, 128, [4, 4], in_flight=3, shuffle=False, seed=2, requests=rq,
                                 driver=driver, formats=formats)
        for i, batch in enumerate(loader):
            lone.run(ids[i * 128:(i + 1) * 128], 2 * 7919 * 10 + i)
            want = lone.result()
            if formats:
                for p, q in zip(batch["blocks"], want["blocks"]):
                    assert sorted(p["formats"]) == sorted(q["formats"]) and "csr_eids" in p["formats"]
                    for k, v in p["formats"].items():
                        assert v == q["formats"][k] if k == "num_edges" else torch.equal(v, q["formats"][k]), k
            assert batch["request_sizes"] == want["request_sizes"] and sum(batch["request_sizes"]) == want["sizes"][-1]
            assert batch["request_sizes"][0] > 0 and sum(batch["request_sizes"][1:]) > 0
            assert torch.equal(batch["request_ids"], want["request_ids"])
            assert torch.equal(batch["request_perm"], want["request_perm"])
            assert torch.equal(batch["features"], want["features"]) and torch.equal(batch["input_nodes"], want["input_nodes"])
        assert i == 9


@pytest.mark.parametrize("layout", [[0], [0, 0, 0, 0, 0], [0, 1, 0], [0, 1, 2, 3, 0, 1, 2]])
def test_epoch_driver_slot_layouts_and_restart(capi, layout):
    """The library's epoch driver on its own: slots spread unevenly over streams (every slot with a table of its own),
    a consumer that keeps every batch busy on its stream before releasing it, an epoch begun while the one before
    is half consumed, and one ended early; every batch equals a lone pipeline's for the same seeds and key."""
    import torch

    from apt_amd.pipeline import MiniBatchPipeline
    g, store, table = _setup(capi)
    B, hops = 96, [4, 3]
    streams = [torch.cuda.Stream() for _ in range(max(layout) + 1)]
    pipes = [MiniBatchPipeline(g, store, B, hops) for _ in layout]
    lone = MiniBatchPipeline(g, store, B, hops)
    drv = capi.EpochDriver(pipes, [streams[k] for k in layout])
    gen = torch.Generator(device="cuda")
    gen.manual_seed(5)
    sink = torch.zeros(1 << 20, device="cuda")

    def epoch(num, key0, consume):
        seeds = torch.randint(0, 30000, (num * B,), generator=gen, device="cuda")
        ready = torch.cuda.Event()
        ready.record()
        drv.begin(seeds, num, key0, ready)
        for i in range(consume):
            k, sizes, rs, fe = drv.next()
            assert k == i % len(layout) and rs is None and fe is None
            pipe = pipes[k]
            pipe.seeds = seeds[i * B:(i + 1) * B]
            got = pipe.result(sizes=sizes)
            for _ in range(3):                           # work on the consumer's stream that reads the slot's buffers
                sink[:got["features"].numel()] += got["features"].reshape(-1)
            kept = (got["input_nodes"].clone(), got["features"].clone(), [b["relabeled"].clone() for b in got["blocks"]])
            drv.release()
            lone.run(seeds[i * B:(i + 1) * B], key0 + i)
            want = lone.result()
            assert sizes[:len(hops) + 1] == want["sizes"] and torch.equal(kept[0], want["input_nodes"])
            assert torch.equal(kept[1], want["features"]) and torch.equal(kept[1], table[kept[0]])
            for a, b in zip(kept[2], want["blocks"]):
                assert torch.equal(a, b["relabeled"])

    epoch(9, 1000, 9)
    epoch(7, 2000, 3)          # left half consumed: the next begin ends it
    epoch(2 * len(layout) + 1, 3000, 2 * len(layout) + 1)
    drv.end()
    drv.end()                  # ending twice is harmless
    epoch(1, 4000, 1)
    drv.close()


def test_loader_with_frequent_table_refills(capi):
    """The rank table runs out of epochs every other batch (or every batch) when its id field is made as wide as it
    gets: the epoch driver's batches, two buffer sets sharing a stream's table, stay what a lone pipeline with the
    default width builds."""
    import torch

    from apt_amd.loader import MiniBatchLoader
    from apt_amd.pipeline import MiniBatchPipeline
    g, store, table = _setup(capi)
    ids = torch.arange(0, 200 * 24).cuda() % 30000
    lone = MiniBatchPipeline(g, store, 200, [4, 3])
    want = []
    for i in range(24):
        lone.run(ids[i * 200:(i + 1) * 200], 5 * 7919 * 24 + i)          # the loader's key for seed 5, first epoch
        r = lone.result()
        want.append((r["input_nodes"].clone(), r["features"].clone(), [b["relabeled"].clone() for b in r["blocks"]]))
    try:
        for bits in (30, 31):
            capi.check(capi.lib().apt_set_tuning(b"minibatch_payload_bits", bits))
            for in_flight in (1, 4):
                loader = MiniBatchLoader(g, store, ids, 200, [4, 3], in_flight=in_flight, shuffle=False, seed=5, driver="c")
                for i, b in enumerate(loader):
                    assert torch.equal(b["input_nodes"], want[i][0]) and torch.equal(b["features"], want[i][1]), (bits, i)
                    for x, y in zip(b["blocks"], want[i][2]):
                        assert torch.equal(x["relabeled"], y), (bits, in_flight, i)
                assert i == 23
    finally:
        capi.check(capi.lib().apt_set_tuning(b"minibatch_payload_bits", 0))


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


@pytest.mark.parametrize("formats", [False, True, "inner"])
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
                # "inner": CSR for every block but the outermost, whose backward pass (towards the raw features)
                # nobody asks for
                assert blocks[0].formats is not None and ("csr_indptr" in blocks[0].formats) == (formats is True)
                assert "csr_indptr" in blocks[1].formats
            h = l2(blocks[1], l1(blocks[0], batch["features"]))
            loss = torch.nn.functional.cross_entropy(h, labels[batch["output_nodes"]])
            opt.zero_grad()
            loss.backward()
            opt.step()
            losses.append(loss.item())
    assert len(losses) == 4 * 15
    assert np.mean(losses[-10:]) < 0.6 * np.mean(losses[:5]), (losses[:5], losses[-10:])
