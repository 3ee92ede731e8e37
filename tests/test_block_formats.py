"""COO / CSC / CSR emission of a sampled block: oracle pins (no GPU) and GPU parity."""
import numpy as np
import pytest


def _random_block(rng, num_dst, fanout, num_src, hole=0.3, hub=True):
    """Fixed-stride block with -1 holes (anywhere in a row, not only at its end)."""
    r = rng.integers(0, max(num_src, 1), size=num_dst * fanout)
    if hub and num_src > 3:
        r[rng.random(r.size) < 0.2] = 3                      # one source on a fifth of all edges
    r[rng.random(r.size) < hole] = -1
    if num_src == 0:
        r[:] = -1
    return r.astype(np.int64)


def _closed_form(r, num_dst, fanout, num_src):
    keep = np.nonzero(r >= 0)[0]
    row, col = r[keep], keep // max(fanout, 1)
    order = np.argsort(row, kind="stable")
    return dict(num_edges=len(keep), coo_row=row, coo_col=col,
                csc_indptr=np.concatenate([[0], np.cumsum(np.bincount(col, minlength=num_dst))]),
                csr_indptr=np.concatenate([[0], np.cumsum(np.bincount(row, minlength=num_src))]),
                csr_indices=col[order], csr_eids=order)


def _same(a, b, keys=("coo_row", "coo_col", "csc_indptr", "csr_indptr", "csr_indices", "csr_eids")):
    assert a["num_edges"] == b["num_edges"]
    for k in keys:
        assert np.array_equal(np.asarray(a[k]), np.asarray(b[k])), k


CASES = [(0, 5, 0), (1, 1, 1), (7, 3, 5), (100, 10, 37), (1000, 15, 5000), (257, 16, 70000), (64, 0, 10)]


def test_oracle_block_formats_closed_form(orc):
    rng = np.random.default_rng(0)
    for num_dst, fanout, num_src in CASES:
        r = _random_block(rng, num_dst, fanout, num_src)
        _same(orc.block_formats(r, num_dst, fanout, num_src), _closed_form(r, num_dst, fanout, num_src))
    # scipy agrees on the offsets and on the neighbour sets of a duplicate-free block
    import scipy.sparse as sp
    num_dst, fanout, num_src = 50, 4, 400
    r = rng.permutation(num_src)[:num_dst * fanout].astype(np.int64)
    got = orc.block_formats(r, num_dst, fanout, num_src)
    m = sp.coo_matrix((np.arange(got["num_edges"]) + 1, (got["coo_row"], got["coo_col"])), shape=(num_src, num_dst))
    csr, csc = m.tocsr(), m.tocsc()
    assert np.array_equal(csr.indptr, got["csr_indptr"]) and np.array_equal(csc.indptr, got["csc_indptr"])
    assert np.array_equal(csr.indices, got["csr_indices"]) and np.array_equal(csr.data - 1, got["csr_eids"])
    assert np.array_equal(csc.indices, got["coo_row"][csc.data - 1])          # scipy orders a column by source
    assert np.array_equal(np.sort((csc.data - 1).reshape(num_dst, fanout), axis=1),
                          np.arange(num_dst * fanout).reshape(num_dst, fanout))


@pytest.mark.gpu
def test_gpu_block_formats(orc, capi):
    import torch
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")
    host = lambda d: {k: (v.cpu().numpy() if hasattr(v, "cpu") else v) for k, v in d.items()}
    rng = np.random.default_rng(1)
    big = [(70000, 15, 300000), (5000, 64, 2 ** 24 + 5), (300000, 5, 17),      # 3 / 4 / 1 digit passes
           (10, 2, 3_000_000), (1, 1, 70_000)]                                # a few edges, sources far apart
    for num_dst, fanout, num_src in CASES + big:
        for hole in (0.0, 0.3, 1.0):
            r = _random_block(rng, num_dst, fanout, num_src, hole)
            want = orc.block_formats(r, num_dst, fanout, num_src)
            got = host(capi.block_formats(dev(r) if r.size else torch.empty(0, dtype=torch.int64, device="cuda:0"),
                                          num_dst, fanout, num_src))
            _same(got, want)
    # the scan launches that large inputs take, forced on small ones; then two inputs large enough by themselves
    capi.check(capi.lib().apt_set_tuning(b"block_fused_scan", 0))
    try:
        for num_dst, fanout, num_src in [(7, 3, 5), (70000, 15, 300000), (5000, 64, 2 ** 24 + 5)]:
            r = _random_block(rng, num_dst, fanout, num_src)
            _same(host(capi.block_formats(dev(r), num_dst, fanout, num_src)), orc.block_formats(r, num_dst, fanout, num_src))
    finally:
        capi.check(capi.lib().apt_set_tuning(b"block_fused_scan", 1))
    for num_dst, fanout, num_src in [(600000, 15, 3000000), (1200000, 15, 70000)]:
        r = _random_block(rng, num_dst, fanout, num_src)
        _same(host(capi.block_formats(dev(r), num_dst, fanout, num_src)), orc.block_formats(r, num_dst, fanout, num_src))
    # no CSR asked for
    r = _random_block(rng, 1000, 7, 900)
    got = host(capi.block_formats(dev(r), 1000, 7, 900, want_csr=False))
    _same(got, orc.block_formats(r, 1000, 7, 900), keys=("coo_row", "coo_col", "csc_indptr"))
    # device-side destination count: buffers at the upper bound, rows past the count are empty
    num_dst, fanout, num_src = 20000, 10, 50000
    r = _random_block(rng, num_dst, fanout, num_src)
    fmt = capi.BlockFormats(num_dst, fanout, num_src)
    for real in (20000, 12345, 1, 0):                        # reuse of the buffers, shrinking
        cnt = torch.tensor([real], dtype=torch.int64, device="cuda:0")
        fmt.emit(dev(r), cnt)
        want = orc.block_formats(r[:real * fanout], real, fanout, num_src)
        e = want["num_edges"]
        assert int(fmt.num_edges.item()) == e
        assert np.array_equal(fmt.csc_indptr.cpu().numpy(), np.concatenate([want["csc_indptr"], np.full(num_dst - real, e)]))
        assert np.array_equal(fmt.csr_indptr.cpu().numpy(), want["csr_indptr"])
        _same(host(fmt.narrow(num_dst=real)), want)


@pytest.mark.gpu
def test_gpu_pipeline_blocks_in_all_formats(orc, capi):
    """The fused driver's blocks, emitted with device-side sizes, equal the
    oracle's formats of the oracle's blocks."""
    import torch
    from helpers import small_graph
    from apt_amd.pipeline import MiniBatchPipeline
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")
    indptr, indices = small_graph(20000, 6, seed=3)
    feats = torch.randn(20000, 32, device="cuda:0")
    graph = capi.Graph(dev(indptr), dev(indices))
    rng = np.random.default_rng(5)
    for use_graph, what in ((False, True), (True, True), (False, "csc"), (True, "csc")):
        pipe = MiniBatchPipeline(graph, capi.FeatStore(feats), 256, [4, 8, 12], formats=what, use_graph=use_graph)
        for key in (77, 78, 79):                              # buffers and streams are reused batch after batch
            seeds = rng.permutation(20000)[:256]
            pipe.run(dev(seeds), key)
            res = pipe.result()
            inp, blocks = orc.sample_blocks(orc.Graph(indptr, indices), seeds, [4, 8, 12], False, key)
            assert len(res["blocks"]) == 3
            assert torch.equal(res["features"], feats[torch.from_numpy(inp).to("cuda:0")])
            for got, want in zip(res["blocks"], blocks):
                f = got["formats"]
                num_dst, num_src = len(want["seeds"]), len(want["unique"])
                ref = orc.block_formats(want["relabeled"], num_dst, want["fanout"], num_src)
                assert f["csc_indptr"].numel() == num_dst + 1
                if what == "csc":
                    assert "csr_indptr" not in f
                    _same({k: (v.cpu().numpy() if hasattr(v, "cpu") else v) for k, v in f.items()}, ref,
                          keys=("coo_row", "coo_col", "csc_indptr"))
                    continue
                assert f["csr_indptr"].numel() == num_src + 1
                _same({k: (v.cpu().numpy() if hasattr(v, "cpu") else v) for k, v in f.items()}, ref)
