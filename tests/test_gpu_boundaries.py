"""Sizes on and around the tile boundaries of the kernels (workgroup tiles of
1024 / 2048 / 4096 items, wavefronts of 64), host-side and device-side counts:
every entry point against the oracle."""
import numpy as np
import pytest
import torch

from helpers import small_graph

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
SIZES = [1, 63, 64, 65, 255, 256, 257, 1023, 1024, 1025, 2047, 2048, 2049, 4095, 4096, 4097, 8191, 8193, 16385]


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def host(t):
    return t.cpu().numpy()


def test_relabel_sizes(orc, capi):
    rng = np.random.default_rng(0)
    for n in SIZES:
        for ns in (0, 1, n // 3, n):
            seeds = rng.integers(0, max(n // 2, 2), size=ns)
            nbrs = rng.integers(0, max(n // 2, 2), size=n - ns)
            nbrs[rng.random(nbrs.size) < 0.05] = -1
            wu, wr = orc.relabel(seeds, nbrs)
            u, r, cnt = capi.relabel(dev(seeds.astype(np.int64)), dev(nbrs.astype(np.int64)))
            assert cnt == len(wu) and np.array_equal(host(u), wu) and np.array_equal(host(r), wr), (n, ns)


def test_bucket_and_format_sizes(orc, capi):
    rng = np.random.default_rng(1)
    min_vids = np.array([0, 100, 250, 600, 1000], dtype=np.int64)
    for n in SIZES:
        ids = rng.integers(0, 1000, size=n)
        want = orc.cluster_permute(ids, min_vids, 4, 0, 2, 0, 4)
        got = capi.cluster_permute(dev(ids), dev(min_vids), 4, 0, 2, 0, 4)
        for a, b in zip(got, want):
            assert np.array_equal(host(a), b), n
        # a block with n slots: fanout 1 and fanout 7 (ragged last tile either way)
        for fanout in (1, 7):
            num_dst = max(n // fanout, 1)
            num_src = max(n // 2, 1)
            rel = rng.integers(0, num_src, size=num_dst * fanout).astype(np.int64)
            rel[rng.random(rel.size) < 0.3] = -1
            ref = orc.block_formats(rel, num_dst, fanout, num_src)
            f = capi.block_formats(dev(rel), num_dst, fanout, num_src)
            for k in ("coo_row", "coo_col", "csc_indptr", "csr_indptr", "csr_indices", "csr_eids"):
                assert np.array_equal(host(f[k]), ref[k]), (n, fanout, k)


def test_sample_and_gather_sizes(orc, capi):
    rng = np.random.default_rng(2)
    indptr, indices = small_graph(3000, 20, seed=3)
    og, dg = orc.Graph(indptr, indices), capi.Graph(dev(indptr), dev(indices))
    feats = rng.standard_normal((3000, 24)).astype(np.float32)
    ofs, dfs = orc.FeatStore(feats), capi.FeatStore(dev(feats))
    for n in SIZES:
        frontier = rng.integers(0, 3000, size=n)
        for fanout, replace in ((15, False), (3, True)):
            wn, wc = orc.sample_neighbors(og, frontier, fanout, replace, 5, 1)
            gn, gc = capi.sample_neighbors(dg, dev(frontier), fanout, replace, 5, 1)
            assert np.array_equal(host(gn), wn) and np.array_equal(host(gc), wc), (n, fanout)
        # the same rows with the count on the device and a larger host-side bound
        bound = dev(np.concatenate([frontier, rng.integers(0, 3000, size=777)]))
        cnt = torch.tensor([n], dtype=torch.int64, device=DEV)
        gn, gc = capi.sample_neighbors(dg, bound, 15, False, 5, 1, num_frontier_dev=cnt)
        wn, wc = orc.sample_neighbors(og, frontier, 15, False, 5, 1)
        assert np.array_equal(host(gn)[:n * 15], wn) and np.array_equal(host(gc)[:n], wc), n
        want, _ = orc.gather_rows(ofs, frontier)
        assert np.array_equal(host(capi.gather_rows(dfs, dev(frontier))), want), n
        out = torch.zeros((n + 777, 24), device=DEV)
        capi.gather_rows(dfs, bound, num_index_dev=cnt, out=out)
        assert np.array_equal(host(out)[:n], want) and not host(out)[n:].any(), n
