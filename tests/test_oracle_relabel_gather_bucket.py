"""Pins the oracle's relabel, gather, pack/unpack and bucketing against numpy
closed forms (no GPU)."""
import numpy as np
import pytest

from helpers import (bucket_closed_form, first_occurrence_unique, gather_closed_form,
                     reqs_closed_form)


def _check_relabel(orc, seeds, nbrs):
    uniq, rel = orc.relabel(seeds, nbrs)
    wu, wr = first_occurrence_unique(seeds, nbrs)
    assert np.array_equal(uniq, wu)
    assert np.array_equal(rel, wr)


def test_relabel_random(orc):
    rng = np.random.default_rng(0)
    for ns, f, hi in [(1, 1, 5), (10, 3, 20), (1024, 5, 3000), (6144, 10, 100000)]:
        seeds = rng.permutation(hi)[:ns]
        nbrs = rng.integers(0, hi, size=ns * f)
        _check_relabel(orc, seeds, nbrs)


def test_relabel_specials(orc):
    rng = np.random.default_rng(1)
    _check_relabel(orc, np.array([5, 9, 7]), np.array([], dtype=np.int64))       # no neighbours
    _check_relabel(orc, np.array([], dtype=np.int64), np.array([3, 3, 1, 3]))    # no seeds
    _check_relabel(orc, np.array([4]), np.full(50, 4))                            # all equal
    _check_relabel(orc, np.array([2, 2, 8, 2]), np.array([8, 1, 2, 1]))           # duplicate seeds
    _check_relabel(orc, np.arange(512), rng.integers(0, 512, 512))                # n power of two
    big = 111_059_956
    _check_relabel(orc, np.array([big - 1, 0, big - 2]), rng.integers(big - 50, big, 64))
    # ids that collide under key & (cap-1) in the reference's table
    _check_relabel(orc, np.arange(8) * 4096, (rng.integers(0, 8, 100) * 4096))
    # padding passes through
    uniq, rel = orc.relabel(np.array([3, 1]), np.array([1, -1, 7, -1, 3]))
    assert uniq.tolist() == [3, 1, 7] and rel.tolist() == [1, -1, 2, -1, 0]


def test_relabel_threaded_variant(orc):
    """Beyond 4096 items and with more than one thread the oracle inserts
    concurrently (CAS + atomic minimum, as the reference's kernels do): the same
    closed form must hold, whatever the interleaving."""
    rng = np.random.default_rng(2)
    orc.set_threads(4)
    try:
        for rep in range(5):
            for ns, f, hi in [(4096, 1, 5000), (6144, 10, 100000), (3000, 15, 300), (70000, 15, 2_000_000)]:
                seeds = rng.integers(0, hi, size=ns)                       # repeated seeds too
                nbrs = rng.integers(0, hi, size=ns * f)
                nbrs[rng.random(nbrs.size) < 0.1] = -1
                _check_relabel(orc, seeds, nbrs)
        uniq, rel = orc.relabel(np.array([4]), np.full(9000, 4))          # every item the same key
        assert uniq.tolist() == [4] and not rel.any()
    finally:
        orc.set_threads(1)


@pytest.mark.parametrize("dtype,dim", [(np.float32, 128), (np.float32, 100), (np.uint16, 128),
                                       (np.float32, 7), (np.uint16, 5)])
def test_gather_identity(orc, dtype, dim):
    rng = np.random.default_rng(2)
    table = rng.integers(0, 60000, size=(500, dim)).astype(dtype)
    idx = rng.integers(0, 500, size=777)
    st = orc.FeatStore(table)
    out, miss = orc.gather_rows(st, idx)
    assert miss == 0 and np.array_equal(out, table[idx])
    out, miss = orc.gather_rows(st, np.array([], dtype=np.int64))
    assert out.shape == (0, dim) and miss == 0


def test_gather_two_tables_window_and_misses(orc):
    rng = np.random.default_rng(3)
    total, nloc, ncache, D, Dr, off = 1000, 300, 80, 24, 8, 12
    local = rng.standard_normal((nloc, D)).astype(np.float32)
    cache = rng.standard_normal((ncache, Dr)).astype(np.float32)
    local_idx = rng.permutation(total)[:nloc]
    # half of the cached ids are also local: the cache wins (src/cache_feats.cc:49-55)
    cached_idx = np.concatenate([local_idx[:40], np.setdiff1d(np.arange(total), local_idx)[:40]])
    pos = np.full(total, -1, dtype=np.int64)
    pos[local_idx] = -np.arange(nloc) - 2
    pos[cached_idx] = np.arange(ncache)
    st = orc.FeatStore(local, cache, pos, col_offset=off, out_dim=Dr)
    idx = np.concatenate([rng.integers(0, total, 2000), [-1, total, total + 7]])
    out, miss = orc.gather_rows(st, idx)
    want, wmiss = gather_closed_form(local, cache, pos, off, Dr, idx)
    assert np.array_equal(out, want) and miss == wmiss and miss > 3
    # precedence spot check
    r = int(cached_idx[0])
    assert np.array_equal(orc.gather_rows(st, [r])[0][0], cache[0])


def test_permute_and_scatter_are_inverse(orc):
    rng = np.random.default_rng(4)
    x = rng.standard_normal((333, 16)).astype(np.float32)
    perm = rng.permutation(333)
    unpacked = orc.permute_rows(x, perm)
    assert np.array_equal(unpacked, x[perm])                      # index_select
    packed = orc.scatter_rows(x, perm)
    want = np.zeros_like(x)
    want[perm] = x                                                # index_select_backward, bijection
    assert np.array_equal(packed, want)
    assert np.array_equal(orc.permute_rows(packed, perm), x)


def test_bucketing_reference_fixture(orc):
    """Inputs of tests/test_shuffle_seeds.cc:19-26 (min_vids = 100*arange(W+1),
    seeds = W*arange(99)+rank); the reference asserts nothing there, the
    expected values come from the closed form."""
    for W in (1, 2, 4, 8):
        for rank in range(W):
            min_vids = 100 * np.arange(W + 1)
            seeds = W * np.arange(99) + rank
            got = orc.cluster_permute(seeds, min_vids, W, 0, rank, 0, W)
            want = bucket_closed_form(seeds, min_vids, W, 0, rank, 0, W)
            for g, w in zip(got, want):
                assert np.array_equal(g, w)
            bs, bo, so, pm = got
            assert np.array_equal(so[pm], seeds)
            assert bs.sum() == 99 and bo[-1] == 99


def test_bucketing_random_and_hybrid(orc):
    rng = np.random.default_rng(5)
    W = 8
    min_vids = np.concatenate([[0], np.sort(rng.integers(1, 10000, W - 1)), [10000]])
    ids = rng.integers(0, 10000, size=5000)
    for (off, rank, beg, end) in [(0, 0, 0, 8), (0, 5, 4, 8), (2, 3, 0, 8), (0, 1, 0, 4)]:
        got = orc.cluster_permute(ids, min_vids, W, off, rank, beg, end)
        want = bucket_closed_form(ids, min_vids, W, off, rank, beg, end)
        for g, w in zip(got, want):
            assert np.array_equal(g, w)
    empty = orc.cluster_permute(np.array([], dtype=np.int64), min_vids, W)
    assert empty[0].sum() == 0 and len(empty[2]) == 0


def test_request_bucketing(orc):
    rng = np.random.default_rng(6)
    W, R, total = 8, 4, 8000
    min_vids = np.arange(W + 1) * 1000
    fm = np.where(rng.random(total) < 0.4, -1, rng.integers(0, 100, total)).astype(np.int64)
    remote_worker_map = np.array([0, 0, 1, 1, 2, 2, 3, 3])
    ids = rng.integers(0, total, size=3000)
    got = orc.cluster_reqs(ids, fm, remote_worker_map, min_vids, W, R)
    want = reqs_closed_form(ids, fm, remote_worker_map, min_vids, W, R)
    for g, w in zip(got, want):
        assert np.array_equal(g, w)
    assert np.array_equal(got[2][got[3]], ids)
