"""Property tests of the oracle's integer functions against numpy closed forms,
on inputs drawn by hypothesis (small, adversarial shapes: empty, all equal,
padding, ids at the range ends).  No GPU."""
import numpy as np
from hypothesis import given, settings
from hypothesis import strategies as st

import oracle as orc
from helpers import bucket_closed_form, first_occurrence_unique

ids = st.lists(st.integers(min_value=-1, max_value=40), max_size=60)
SET = dict(max_examples=150, deadline=None)


@settings(**SET)
@given(seeds=st.lists(st.integers(min_value=0, max_value=40), max_size=20), nbrs=ids)
def test_relabel(seeds, nbrs):
    uniq, rel = orc.relabel(np.array(seeds, dtype=np.int64), np.array(nbrs, dtype=np.int64))
    wu, wr = first_occurrence_unique(np.array(seeds, dtype=np.int64), np.array(nbrs, dtype=np.int64))
    assert np.array_equal(uniq, wu) and np.array_equal(rel, wr)


@settings(**SET)
@given(v=st.lists(st.integers(min_value=0, max_value=99), max_size=80),
       cuts=st.lists(st.integers(min_value=1, max_value=99), min_size=0, max_size=5, unique=True),
       rank=st.integers(0, 5), lo=st.integers(0, 5), span=st.integers(1, 6))
def test_cluster_permute(v, cuts, rank, lo, span):
    min_vids = np.array([0] + sorted(cuts) + [100], dtype=np.int64)
    w = len(min_vids) - 1
    rank, lo = rank % w, lo % w
    hi = min(w, lo + span)
    if not lo <= rank < hi:            # the owner rule folds foreign owners onto the own rank, which must be local
        lo, hi = 0, w
    ids_ = np.array(v, dtype=np.int64)
    got = orc.cluster_permute(ids_, min_vids, w, 0, rank, lo, hi)
    want = bucket_closed_form(ids_, min_vids, w, 0, rank, lo, hi)
    for a, b in zip(got, want):
        assert np.array_equal(a, b)


@settings(**SET)
@given(rows=st.lists(st.lists(st.integers(min_value=-1, max_value=12), min_size=4, max_size=4), max_size=15))
def test_block_formats(rows):
    rel = np.array(rows, dtype=np.int64).reshape(-1)
    num_dst, fanout, num_src = len(rows), 4, 13
    f = orc.block_formats(rel, num_dst, fanout, num_src)
    keep = np.nonzero(rel >= 0)[0]
    row, col = rel[keep], keep // fanout
    order = np.argsort(row, kind="stable")
    assert np.array_equal(f["coo_row"], row) and np.array_equal(f["coo_col"], col)
    assert np.array_equal(f["csc_indptr"], np.concatenate([[0], np.cumsum(np.bincount(col, minlength=num_dst))]))
    assert np.array_equal(f["csr_indptr"], np.concatenate([[0], np.cumsum(np.bincount(row, minlength=num_src))]))
    assert np.array_equal(f["csr_indices"], col[order]) and np.array_equal(f["csr_eids"], order)


@settings(**SET)
@given(deg=st.lists(st.integers(min_value=0, max_value=6), min_size=1, max_size=12),
       pick=st.lists(st.integers(min_value=-2, max_value=14), max_size=20), begin=st.integers(0, 3))
def test_csr_select_rows_and_counts(deg, pick, begin):
    indptr = np.concatenate([[0], np.cumsum(deg)]).astype(np.int64)
    indices = np.arange(indptr[-1], dtype=np.int64) * 3 + 1
    g = orc.Graph(indptr, indices, row_begin=begin, num_total_nodes=begin + len(deg) + 3)
    rows = np.array(pick, dtype=np.int64)
    ip, ix = orc.csr_select_rows(g, rows)
    want = [indices[indptr[r - begin]:indptr[r - begin + 1]] if 0 <= r - begin < len(deg) else indices[:0] for r in rows]
    assert np.array_equal(np.diff(ip), [len(w) for w in want]) and ip[0] == 0
    assert np.array_equal(ix, np.concatenate(want) if want else indices[:0])
    freq = np.zeros(10, dtype=np.int64)
    orc.count_ids(rows, freq)
    assert np.array_equal(freq, np.bincount(rows[(rows >= 0) & (rows < 10)], minlength=10))


@settings(**SET)
@given(src=st.lists(st.integers(min_value=0, max_value=99), min_size=0, max_size=40),
       cuts=st.lists(st.integers(min_value=1, max_value=99), min_size=0, max_size=4, unique=True),
       fanout=st.integers(1, 5))
def test_virtual_nodes(src, cuts, fanout):
    min_vids = np.array([0] + sorted(cuts) + [100], dtype=np.int64)
    w = len(min_vids) - 1
    s = np.array(src[:len(src) // fanout * fanout], dtype=np.int64)
    nd = len(s) // fanout
    got = orc.map_to_vir(s, fanout, min_vids, w, num_dst=nd)
    owner = np.searchsorted(min_vids[1:w], s, side="right")
    assert np.array_equal(got, owner * nd + np.arange(len(s)) // fanout)
    vs = np.sort(got)
    off = orc.vir_send_offset(w, nd, vs, np.unique(vs), False)
    assert np.array_equal(off[:w + 1], np.searchsorted(vs, np.arange(w + 1) * nd, "left"))
    assert np.array_equal(off[w + 1:], np.searchsorted(np.unique(vs), np.arange(1, w + 1) * nd, "left"))
