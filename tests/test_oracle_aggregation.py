"""Pins the oracle's SpMM / SDDMM against numpy closed forms (no GPU)."""
import numpy as np


def _block(rng, n_dst=300, fanout=7, n_src=900):
    col = np.repeat(np.arange(n_dst), fanout)
    row = rng.integers(0, n_src, size=len(col))
    keep = rng.random(len(col)) < 0.9                       # ragged rows, still grouped by destination
    return row[keep], col[keep], n_src, n_dst


def test_spmm_modes_closed_form(orc):
    rng = np.random.default_rng(0)
    row, col, n_src, n_dst = _block(rng)
    x = rng.standard_normal((n_src, 24)).astype(np.float32)
    xe = rng.standard_normal((len(row), 24)).astype(np.float32)
    want = np.zeros((n_dst, 24)); np.add.at(want, col, x[row].astype(np.float64))
    assert np.allclose(orc.spmm_sum(0, row, col, x, n_dst), want, rtol=1e-6, atol=1e-6)
    want = np.zeros((n_dst, 24)); np.add.at(want, col, xe.astype(np.float64))
    assert np.allclose(orc.spmm_sum(1, row, col, xe, n_dst), want, rtol=1e-6, atol=1e-6)
    want = np.zeros((n_dst, 24)); np.add.at(want, col, x[row].astype(np.float64) * xe)
    assert np.allclose(orc.spmm_sum(2, row, col, x, n_dst, edata=xe), want, rtol=1e-6, atol=1e-6)
    # a table of ones sums to the in-degree
    ones = np.ones((n_src, 3), dtype=np.float32)
    assert np.array_equal(orc.spmm_sum(0, row, col, ones, n_dst)[:, 0], np.bincount(col, minlength=n_dst))


def test_spmm_segments(orc):
    """Two concatenated blocks with their own input / output bases
    (reference src/cuda/spmm.cu:21-24)."""
    rng = np.random.default_rng(1)
    r1, c1, s1, d1 = _block(rng, 50, 4, 120)
    r2, c2, s2, d2 = _block(rng, 70, 3, 90)
    row, col = np.concatenate([r1, r2]), np.concatenate([c1, c2])
    x = rng.standard_normal((s1 + s2, 8)).astype(np.float32)
    got = orc.spmm_sum(0, row, col, x, d1 + d2, coo_offset=[0, len(r1), len(row)], input_offset=[0, s1],
                       output_offset=[0, d1, d1 + d2])
    want = np.zeros((d1 + d2, 8))
    np.add.at(want, c1, x[r1].astype(np.float64))
    np.add.at(want, d1 + c2, x[s1 + r2].astype(np.float64))
    assert np.allclose(got, want, rtol=1e-6, atol=1e-6)


def test_sddmm_closed_form(orc):
    rng = np.random.default_rng(2)
    row, col, n_src, n_dst = _block(rng)
    lhs = rng.standard_normal((n_src, 16)).astype(np.float32)
    rhs = rng.standard_normal((n_dst, 16)).astype(np.float32)
    assert np.array_equal(orc.sddmm(0, row, col, lhs, rhs), lhs[row] + rhs[col])
    assert np.array_equal(orc.sddmm(1, row, col, lhs, rhs), lhs[row] * rhs[col])


def _ell_block(rng, n_dst, fanout, n_src, distinct=False, hole=0.25):
    """Fixed-stride block; distinct=True: no source twice in a row."""
    if distinct:
        nbr = np.stack([rng.permutation(n_src)[:fanout] for _ in range(n_dst)]).astype(np.int64)
    else:
        nbr = rng.integers(0, n_src, size=(n_dst, fanout)).astype(np.int64)
    nbr[rng.random(nbr.shape) < hole] = -1
    nbr[0, :] = -1                                         # a destination without neighbours
    nbr[1, 1:] = -1                                        # ... and with at most one
    return nbr.reshape(-1)


def test_gat_scores_and_block_pins(orc):
    from scipy.special import softmax
    rng = np.random.default_rng(7)
    n_dst, fanout, n_src, heads, dim = 40, 6, 90, 3, 5
    ft = rng.standard_normal((n_src, heads, dim)).astype(np.float32)
    al, ar = rng.standard_normal((2, heads, dim)).astype(np.float32)
    el, er = orc.gat_scores(ft, al), orc.gat_scores(ft[:n_dst], ar)
    assert np.allclose(el, np.einsum("nhd,hd->nh", ft.astype(np.float64), al), rtol=1e-6, atol=1e-6)
    # (1) dense statement with a library softmax: duplicate-free rows, so A[d, s] is one edge
    nbr = _ell_block(rng, n_dst, fanout, n_src, distinct=True)
    out, attn = orc.gat_block(nbr, n_dst, fanout, ft, el, er, 0.2, want_attn=True)
    mask = np.zeros((n_dst, n_src), dtype=bool)
    rows = np.repeat(np.arange(n_dst), fanout)
    mask[rows[nbr >= 0], nbr[nbr >= 0]] = True
    for h in range(heads):
        z = el[None, :, h].astype(np.float64) + er[:, None, h]
        z = np.where(z > 0, z, 0.2 * z)
        z[~mask] = -np.inf
        some = mask.any(1)
        a = np.zeros_like(z)
        a[some] = softmax(z[some], axis=1)
        assert np.allclose(out[:, h, :], a @ ft[:, h, :].astype(np.float64), rtol=1e-6, atol=1e-6)
        got_a = attn.reshape(n_dst, fanout, heads)[:, :, h]
        assert np.allclose(got_a[nbr.reshape(n_dst, fanout) >= 0], a[rows[nbr >= 0], nbr[nbr >= 0]], rtol=1e-6, atol=1e-7)
    assert np.all(out[0] == 0) and np.all(attn.reshape(n_dst, fanout, heads)[0] == 0)
    # (2) equal logits -> plain mean over the row's edges (duplicates allowed), which the SpMM oracle computes
    nbr = _ell_block(rng, n_dst, fanout, n_src)
    zeros_s, zeros_d = np.zeros((n_src, heads), np.float32), np.zeros((n_dst, heads), np.float32)
    out = orc.gat_block(nbr, n_dst, fanout, ft, zeros_s, zeros_d)
    keep = nbr >= 0
    mean = orc.spmm_sum(0, nbr[keep], rows[keep], ft.reshape(n_src, -1), n_dst)
    cnt = np.maximum(np.bincount(rows[keep], minlength=n_dst), 1)[:, None]
    assert np.allclose(out.reshape(n_dst, -1), mean / cnt, rtol=1e-6, atol=1e-6)
    # (3) attention sums to one per destination and head; a lone neighbour passes through
    out, attn = orc.gat_block(nbr, n_dst, fanout, ft, el, er, 0.2, want_attn=True)
    sums = attn.reshape(n_dst, fanout, heads).sum(1)
    has = np.bincount(rows[keep], minlength=n_dst) > 0
    assert np.allclose(sums[has], 1, atol=1e-6) and np.all(sums[~has] == 0)
    if nbr[fanout] >= 0:
        assert np.allclose(out[1], ft[nbr[fanout]], rtol=1e-6)
    # (4) softmax is shift invariant on the positive side: logits all > 0 stay linear under + c on er
    big_l, big_r = np.abs(el) + 1, np.abs(er) + 1
    a = orc.gat_block(nbr, n_dst, fanout, ft, big_l, big_r)
    b = orc.gat_block(nbr, n_dst, fanout, ft, big_l, big_r + 3.5)
    assert np.allclose(a, b, rtol=1e-5, atol=1e-6)
    # (5) the slope matters only below zero
    neg_l, neg_r = -np.abs(el) - 1, -np.abs(er) - 1
    a = orc.gat_block(nbr, n_dst, fanout, ft, neg_l, neg_r, 0.2)
    b = orc.gat_block(nbr, n_dst, fanout, ft, (0.2 * neg_l).astype(np.float32), (0.2 * neg_r).astype(np.float32), 1.0)
    assert np.allclose(a, b, rtol=1e-5, atol=1e-6)


def test_spmm_csr_is_the_sparse_matrix_product(orc):
    """Row-owned SpMM over CSR = scipy's CSR matrix times the dense features, per
    head with the edge weights as the matrix data (float64); rows without edges are
    zero; the second sum is the matrix times a column of ones."""
    import scipy.sparse as sp
    rng = np.random.default_rng(5)
    rows, n_x, heads, hd = 400, 150, 3, 8
    deg = rng.integers(0, 6, rows)
    deg[7] = 700                                              # a hub row
    deg[11] = 0
    indptr = np.concatenate([[0], np.cumsum(deg)])
    E = int(indptr[-1])
    indices = rng.integers(0, n_x, E)
    eids = rng.permutation(E)
    x = rng.standard_normal((n_x, heads * hd)).astype(np.float32)
    scale = rng.random(n_x).astype(np.float32) + 0.5
    w = rng.standard_normal((E, heads)).astype(np.float32)
    w2 = rng.standard_normal((E, heads)).astype(np.float32)
    # plain sum
    A = sp.csr_matrix((np.ones(E), indices, indptr), shape=(rows, n_x))
    got = orc.spmm_csr(indptr, indices, x)
    assert np.allclose(got, A @ x.astype(np.float64), rtol=1e-6, atol=1e-6) and not got[11].any()
    # scaled columns (the mean's backward)
    got = orc.spmm_csr(indptr, indices, x, col_scale=scale)
    assert np.allclose(got, A @ (x.astype(np.float64) * scale[:, None]), rtol=1e-6, atol=1e-6)
    # per-head edge weights addressed through edge ids, and the second sum
    got, got2 = orc.spmm_csr(indptr, indices, x, eids=eids, head_weights=w, head_weights2=w2, heads=heads)
    for h in range(heads):
        Ah = sp.csr_matrix((w[eids, h].astype(np.float64), indices, indptr), shape=(rows, n_x))
        assert np.allclose(got[:, h * hd:(h + 1) * hd], Ah @ x[:, h * hd:(h + 1) * hd].astype(np.float64),
                           rtol=1e-5, atol=1e-5)
        want2 = np.add.reduceat(np.concatenate([w2[eids, h].astype(np.float64), [0.0]]), indptr[:-1]) * (deg > 0)
        assert np.allclose(got2[:, h], want2, rtol=1e-5, atol=1e-5)
