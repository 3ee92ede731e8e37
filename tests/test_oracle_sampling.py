"""Pins the CPU oracle's RNG and sampler (no GPU).

Philox4x32-10 against published known-answer vectors; the sampler against
closed forms, invariants, brute force and chi-square tests.
"""
import itertools

import numpy as np
import pytest
from scipy import stats

from helpers import small_graph, special_graph

# Random123 kat_vectors (philox4x32 10 rounds): counter, key, expected
KAT = [
    ([0, 0, 0, 0], [0, 0], [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]),
    ([0xffffffff] * 4, [0xffffffff] * 2, [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]),
    ([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], [0xa4093822, 0x299f31d0],
     [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1]),
    # rocRAND's host implementation of the same generator, seed=2^64-1,
    # subsequence=2^64-1, offset 0 (counter words 2,3 hold the subsequence)
    ([0, 0, 0xffffffff, 0xffffffff], [0xffffffff] * 2,
     [0x3d3be307, 0x716983d6, 0x70094bed, 0x36c3cf91]),
]


@pytest.mark.parametrize("ctr,key,want", KAT)
def test_philox_known_answers(orc, ctr, key, want):
    assert [int(x) for x in orc.philox4x32_10(ctr, key)] == want


def test_draw64_layout(orc):
    # counter = (node lo, node hi, hop, slot), key = (seed lo, seed hi),
    # value = word0 | word1 << 32
    seed, node, hop, slot = 0x0123456789abcdef, (5 << 32) | 77, 2, 9
    o = orc.philox4x32_10([77, 5, 2, 9], [0x89abcdef, 0x01234567])
    assert orc.draw64(seed, node, hop, slot) == int(o[0]) | (int(o[1]) << 32)


def test_bounded_is_mulhi(orc):
    rng = np.random.default_rng(0)
    for _ in range(200):
        r = int(rng.integers(0, 2**63)) * 2 + int(rng.integers(0, 2))
        n = int(rng.integers(1, 2**40))
        assert orc.bounded(r, n) == (r * n) >> 64
    assert orc.bounded(2**64 - 1, 7) == 6
    assert orc.bounded(0, 7) == 0


def test_whole_row_when_fanout_covers_degree(orc):
    indptr, indices, degs = special_graph()
    g = orc.Graph(indptr, indices)
    frontier = np.arange(len(degs))
    for fanout in (5, 16, 64):
        nbr, cnt = orc.sample_neighbors(g, frontier, fanout, False, 11, 0)
        nbr = nbr.reshape(len(degs), fanout)
        for v, d in enumerate(degs):
            assert cnt[v] == min(d, fanout)
            if d <= fanout:
                row = indices[indptr[v]:indptr[v + 1]]
                assert np.array_equal(nbr[v, :d], row)          # CSR order
                assert np.all(nbr[v, d:] == -1)


@pytest.mark.parametrize("replace", [False, True])
def test_invariants(orc, replace):
    indptr, indices = small_graph(3000, 14, seed=3)
    g = orc.Graph(indptr, indices)
    rng = np.random.default_rng(1)
    frontier = rng.permutation(3000)[:1024]
    fanout = 10
    nbr, cnt = orc.sample_neighbors(g, frontier, fanout, replace, 99, 1)
    nbr = nbr.reshape(-1, fanout)
    for i, v in enumerate(frontier):
        row = indices[indptr[v]:indptr[v + 1]]
        deg = len(row)
        k = int(cnt[i])
        if replace:
            assert k == (fanout if deg > 0 else 0)
        else:
            assert k == min(fanout, deg)
            # graph is deduplicated, so distinct positions <=> distinct ids
            assert len(set(nbr[i, :k].tolist())) == k
        assert np.all(np.isin(nbr[i, :k], row))                  # true neighbours
        assert np.all(nbr[i, k:] == -1)


def test_keyed_by_node_not_by_position(orc):
    indptr, indices = small_graph(1500, 20, seed=5)
    g = orc.Graph(indptr, indices)
    frontier = np.arange(0, 1500, 3)
    a, ca = orc.sample_neighbors(g, frontier, 7, False, 5, 2)
    perm = np.random.default_rng(2).permutation(len(frontier))
    b, cb = orc.sample_neighbors(g, frontier[perm], 7, False, 5, 2)
    assert np.array_equal(a.reshape(-1, 7)[perm], b.reshape(-1, 7))
    assert np.array_equal(ca[perm], cb)
    # different hop or seed -> different draws somewhere
    c, _ = orc.sample_neighbors(g, frontier, 7, False, 5, 3)
    d, _ = orc.sample_neighbors(g, frontier, 7, False, 6, 2)
    assert not np.array_equal(a, c) and not np.array_equal(a, d)


def test_position_map_and_row_range(orc):
    indptr, indices = small_graph(800, 10, seed=8)
    n = 800
    plain = orc.Graph(indptr, indices)
    # cache rows 0,10,20,... as a second table; the map sends them there
    cached = np.arange(0, n, 10)
    c_indptr = np.zeros(len(cached) + 1, dtype=np.int64)
    c_indptr[1:] = np.cumsum(indptr[cached + 1] - indptr[cached])
    c_indices = np.concatenate([indices[indptr[v]:indptr[v + 1]] for v in cached])
    pos = -np.arange(n, dtype=np.int64) - 2                      # ENCODE_ID(v)
    pos[cached] = np.arange(len(cached))
    mapped = orc.Graph(indptr, indices, cached_indptr=c_indptr, cached_indices=c_indices,
                       adj_pos_map=pos)
    f = np.arange(n)
    for replace in (False, True):
        a = orc.sample_neighbors(plain, f, 6, replace, 3, 0)
        b = orc.sample_neighbors(mapped, f, 6, replace, 3, 0)
        assert np.array_equal(a[0], b[0]) and np.array_equal(a[1], b[1])
    # a partition that owns rows [200, 500): everything else has no adjacency
    part = orc.Graph(indptr[200:501] - indptr[200], indices[indptr[200]:indptr[500]], row_begin=200)
    a = orc.sample_neighbors(plain, f, 6, False, 3, 0)
    b = orc.sample_neighbors(part, f, 6, False, 3, 0)
    inside = (f >= 200) & (f < 500)
    assert np.array_equal(a[0].reshape(-1, 6)[inside], b[0].reshape(-1, 6)[inside])
    assert np.all(b[1][~inside] == 0) and np.all(b[0].reshape(-1, 6)[~inside] == -1)
    # padding / out-of-range ids
    c = orc.sample_neighbors(plain, np.array([-1, n, n + 5, 3]), 4, False, 3, 0)
    assert np.all(c[1][:3] == 0)


def test_subsets_uniform_bruteforce(orc):
    """deg=6, k=3: all 20 subsets equally likely (chi-square over 40000 keys)."""
    deg, k, trials = 6, 3, 40000
    subsets = {s: 0 for s in itertools.combinations(range(deg), k)}
    for node in range(trials):
        pos = orc.sample_positions(deg, k, False, 1234, node, 0)
        subsets[tuple(sorted(pos.tolist()))] += 1
    obs = np.array(list(subsets.values()))
    assert obs.sum() == trials and np.all(obs > 0)
    p = stats.chisquare(obs).pvalue
    assert p > 1e-4, p


@pytest.mark.parametrize("deg,k", [(16, 15), (17, 5), (100, 10), (1000, 15)])
def test_positions_uniform_without_replacement(orc, deg, k):
    trials = 20000
    hist = np.zeros(deg, dtype=np.int64)
    for node in range(trials):
        pos = orc.sample_positions(deg, k, False, 77, node, 1)
        assert len(set(pos.tolist())) == k and pos.min() >= 0 and pos.max() < deg
        hist[pos] += 1
    p = stats.chisquare(hist).pvalue
    assert p > 1e-4, p


def test_positions_uniform_with_replacement(orc):
    deg, k, trials = 37, 8, 20000
    hist = np.zeros(deg, dtype=np.int64)
    slot_hist = np.zeros((k, deg), dtype=np.int64)
    for node in range(trials):
        pos = orc.sample_positions(deg, k, True, 5, node, 0)
        assert len(pos) == k
        hist[pos] += 1
        slot_hist[np.arange(k), pos] += 1
    assert stats.chisquare(hist).pvalue > 1e-4
    for s in range(k):
        assert stats.chisquare(slot_hist[s]).pvalue > 1e-5


def test_multi_hop_driver_structure(orc):
    indptr, indices = small_graph(4000, 15, seed=9)
    g = orc.Graph(indptr, indices)
    seeds = np.random.default_rng(4).permutation(4000)[:256]
    hops = [5, 10]                                               # from the seeds outward
    input_nodes, blocks = orc.sample_blocks(g, seeds, hops, False, 21)
    assert len(blocks) == 2
    inner, outer = blocks[1], blocks[0]                          # blocks are outermost-first
    assert np.array_equal(inner["seeds"], seeds)
    assert np.array_equal(inner["unique"][:len(seeds)], seeds)   # dst nodes are a prefix of src
    assert np.array_equal(outer["seeds"], inner["unique"])
    assert np.array_equal(input_nodes, outer["unique"])
    assert np.array_equal(input_nodes[:len(seeds)], seeds)
    for b in blocks:
        valid = b["neighbors"] >= 0
        assert np.array_equal(b["unique"][b["relabeled"][valid]], b["neighbors"][valid])
        assert valid.sum() == b["counts"].sum()
