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
