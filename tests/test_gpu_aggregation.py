"""SpMM / SDDMM on the GPU vs the oracle: 1e-5 relative in fp32, 1e-2 with
bf16 inputs (accumulation is fp32 in both)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def _block(rng, n_dst, fanout, n_src, shuffle=False):
    col = np.repeat(np.arange(n_dst), fanout)
    row = rng.integers(0, n_src, size=len(col))
    keep = rng.random(len(col)) < 0.9
    row, col = row[keep], col[keep]
    if shuffle:
        p = rng.permutation(len(row))
        row, col = row[p], col[p]
    return row, col


def _close(got, want, rtol):
    scale = np.abs(want).max() + 1e-30
    return np.max(np.abs(got - want)) <= rtol * scale


@pytest.mark.parametrize("dim", [256, 64, 100, 7, 300])
@pytest.mark.parametrize("shuffle", [False, True])
def test_spmm_fp32(orc, capi, dim, shuffle):
    rng = np.random.default_rng(dim)
    n_dst, n_src = 5000, 30000
    row, col = _block(rng, n_dst, 15, n_src, shuffle)
    x = rng.standard_normal((n_src, dim)).astype(np.float32)
    xe = rng.standard_normal((len(row), dim)).astype(np.float32)
    for mode, inp, ed in [(0, x, None), (1, xe, None), (2, x, xe)]:
        want = orc.spmm_sum(mode, row, col, inp, n_dst, edata=ed)
        got = capi.spmm_sum(mode, dev(row), dev(col), dev(inp), n_dst, edata=None if ed is None else dev(ed))
        assert _close(got.cpu().numpy(), want, 1e-5), mode
    if not shuffle:          # edges grouped by destination: independent of scheduling
        a = capi.spmm_sum(0, dev(row), dev(col), dev(x), n_dst)
        b = capi.spmm_sum(0, dev(row), dev(col), dev(x), n_dst)
        assert torch.equal(a, b)


def test_spmm_bf16_and_mean(orc, capi):
    rng = np.random.default_rng(3)
    n_dst, n_src, dim, f = 4000, 20000, 256, 10
    row, col = _block(rng, n_dst, f, n_src)
    x = torch.from_numpy(rng.standard_normal((n_src, dim)).astype(np.float32)).to(DEV).to(torch.bfloat16)
    want = orc.spmm_sum(0, row, col, x.float().cpu().numpy(), n_dst)
    got = capi.spmm_sum(0, dev(row), dev(col), x, n_dst)
    assert _close(got.cpu().numpy(), want, 1e-2)
    assert _close(got.cpu().numpy(), want, 1e-5)            # inputs are exact in fp32, so is the sum
    # GraphSAGE mean = sum / in-degree (reference python/npc/model/sageconv.py:173-174 divides by fanout)
    deg = np.maximum(np.bincount(col, minlength=n_dst), 1)[:, None]
    assert _close((got / dev(deg.astype(np.float32))).cpu().numpy(), want / deg, 1e-2)


def test_spmm_segments_and_empty(orc, capi):
    rng = np.random.default_rng(4)
    r1, c1 = _block(rng, 500, 4, 1200)
    r2, c2 = _block(rng, 700, 3, 900)
    row, col = np.concatenate([r1, r2]), np.concatenate([c1, c2])
    x = rng.standard_normal((2100, 32)).astype(np.float32)
    kw = dict(coo_offset=[0, len(r1), len(row)], input_offset=[0, 1200], output_offset=[0, 500, 1200])
    want = orc.spmm_sum(0, row, col, x, 1200, **kw)
    got = capi.spmm_sum(0, dev(row), dev(col), dev(x), 1200, **{k: dev(np.array(v)) for k, v in kw.items()})
    assert _close(got.cpu().numpy(), want, 1e-5)
    e = dev(np.array([], dtype=np.int64))
    assert capi.spmm_sum(0, e, e, dev(x), 10).abs().sum().item() == 0


@pytest.mark.parametrize("dim", [256, 64, 5])
def test_sddmm(orc, capi, dim):
    rng = np.random.default_rng(dim)
    row, col = _block(rng, 3000, 10, 9000)
    lhs = rng.standard_normal((9000, dim)).astype(np.float32)
    rhs = rng.standard_normal((3000, dim)).astype(np.float32)
    for op in (0, 1):
        want = orc.sddmm(op, row, col, lhs, rhs)
        got = capi.sddmm(op, dev(row), dev(col), dev(lhs), dev(rhs))
        assert np.array_equal(got.cpu().numpy(), want)       # one fp32 operation per element
    lb, rb = dev(lhs).to(torch.bfloat16), dev(rhs).to(torch.bfloat16)
    got = capi.sddmm(1, dev(row), dev(col), lb, rb)
    want = orc.sddmm(1, row, col, lb.float().cpu().numpy(), rb.float().cpu().numpy())
    assert _close(got.cpu().numpy(), want, 1e-2)


def test_aggregation_operators(orc, capi):
    import apt_amd  # noqa: F401
    rng = np.random.default_rng(5)
    row, col = _block(rng, 1000, 5, 4000)
    x = rng.standard_normal((4000, 64)).astype(np.float32)
    y = rng.standard_normal((1000, 64)).astype(np.float32)
    coo = torch.tensor([0, len(row)])
    zero = torch.tensor([0])
    out = torch.ops.npc.spmm_copy_u_sum(dev(row), dev(col), dev(x), coo, zero, torch.tensor([0, 1000]))
    assert _close(out.cpu().numpy(), orc.spmm_sum(0, row, col, x, 1000), 1e-5)
    out = torch.ops.npc.sddmm_u_add_v(dev(row), dev(col), dev(x), dev(y), coo, zero, zero)
    assert np.array_equal(out.cpu().numpy(), orc.sddmm(0, row, col, x, y))


@pytest.mark.parametrize("dim,dtype", [(256, torch.float32), (256, torch.bfloat16), (64, torch.float32),
                                       (100, torch.float32), (7, torch.float32), (1000, torch.float32)])
def test_spmm_block_layout(orc, capi, dim, dtype):
    """The sampler's padded block layout, sum and mean, vs the COO oracle."""
    rng = np.random.default_rng(dim)
    n_dst, n_src, f = 3000, 20000, 15
    nbr = rng.integers(0, n_src, size=(n_dst, f))
    cnt = rng.integers(0, f + 1, size=n_dst)
    nbr[np.arange(f)[None, :] >= cnt[:, None]] = -1                  # ragged rows, some empty
    x = torch.from_numpy(rng.standard_normal((n_src, dim)).astype(np.float32)).to(DEV).to(dtype)
    xh = x.float().cpu().numpy()
    col = np.repeat(np.arange(n_dst), f)
    keep = nbr.reshape(-1) >= 0
    want = orc.spmm_sum(0, nbr.reshape(-1)[keep], col[keep], xh, n_dst)
    got = capi.spmm_block(dev(nbr.reshape(-1)), n_dst, f, x)
    assert _close(got.cpu().numpy(), want, 1e-5)
    got_mean = capi.spmm_block(dev(nbr.reshape(-1)), n_dst, f, x, mean=True)
    assert _close(got_mean.cpu().numpy(), want / np.maximum(cnt, 1)[:, None], 1e-5)
    assert np.all(got.cpu().numpy()[cnt == 0] == 0)
    a = capi.spmm_block(dev(nbr.reshape(-1)), n_dst, f, x)
    assert torch.equal(a, got)                                       # fixed summation order


def _ell(rng, n_dst, fanout, n_src, hole=0.25):
    nbr = rng.integers(0, n_src, size=(n_dst, fanout)).astype(np.int64)
    nbr[rng.random(nbr.shape) < hole] = -1
    nbr[0, :] = -1
    nbr[1, 1:] = -1
    return nbr.reshape(-1)


@pytest.mark.parametrize("heads,dim", [(4, 64), (1, 256), (3, 5), (8, 16), (2, 100), (5, 4), (3, 512), (2, 32)])
def test_gat_fp32(orc, capi, heads, dim):
    rng = np.random.default_rng(heads * 1000 + dim)
    n_dst, fanout, n_src = 3000, 15, 20000
    nbr = _ell(rng, n_dst, fanout, n_src)
    ft = rng.standard_normal((n_src, heads, dim)).astype(np.float32)
    al, ar = (rng.standard_normal((2, heads, dim)) * 0.3).astype(np.float32)
    el, er = capi.gat_scores(dev(ft), dev(al)), capi.gat_scores(dev(ft[:n_dst]), dev(ar))
    assert _close(el.cpu().numpy(), orc.gat_scores(ft, al), 1e-5)
    assert _close(er.cpu().numpy(), orc.gat_scores(ft[:n_dst], ar), 1e-5)
    h_el, h_er = el.cpu().numpy(), er.cpu().numpy()          # same logits into both, so only the block is compared
    want, want_a = orc.gat_block(nbr, n_dst, fanout, ft, h_el, h_er, 0.2, want_attn=True)
    got, got_a = capi.gat_block(dev(nbr), n_dst, fanout, dev(ft), el, er, 0.2, want_attn=True)
    assert _close(got.cpu().numpy(), want, 1e-5)
    assert np.max(np.abs(got_a.cpu().numpy() - want_a)) <= 1e-5
    assert torch.equal(got, capi.gat_block(dev(nbr), n_dst, fanout, dev(ft), el, er, 0.2))   # reproducible
    # device-side row count: rows past it are left alone
    cnt = torch.tensor([1000], dtype=torch.int64, device=DEV)
    part = capi.gat_block(dev(nbr), n_dst, fanout, dev(ft), el, er, 0.2, num_dst_dev=cnt)
    assert torch.equal(part[:1000], got[:1000])


def test_gat_bf16_config5_shape(orc, capi):
    """4 heads x 64, bf16 features, fp32 accumulation: 1e-2 of the oracle on the same (rounded) inputs."""
    rng = np.random.default_rng(11)
    n_dst, fanout, n_src, heads, dim = 4000, 15, 30000, 4, 64
    nbr = _ell(rng, n_dst, fanout, n_src)
    ft16 = torch.from_numpy(rng.standard_normal((n_src, heads, dim)).astype(np.float32)).to(torch.bfloat16)
    ft = ft16.to(torch.float32).numpy()
    al, ar = (rng.standard_normal((2, heads, dim)) * 0.02).astype(np.float32)     # N(0, 0.02) weights
    el, er = capi.gat_scores(ft16.to(DEV), dev(al)), capi.gat_scores(ft16[:n_dst].contiguous().to(DEV), dev(ar))
    assert _close(el.cpu().numpy(), orc.gat_scores(ft, al), 1e-2)
    want = orc.gat_block(nbr, n_dst, fanout, ft, el.cpu().numpy(), er.cpu().numpy(), 0.2)
    got = capi.gat_block(dev(nbr), n_dst, fanout, ft16.to(DEV), el, er, 0.2)
    assert _close(got.cpu().numpy(), want, 1e-2)


def test_spmm_grouped_detection(orc, capi):
    """apt_coo_is_grouped: 1 for a destination-major COO, 0 once two edges are out of
    order; with the flag the sum skips the atomics inside a wavefront's edges and
    gives the oracle's result either way (and the same bits on every call when grouped)."""
    import ctypes
    rng = np.random.default_rng(31)
    row, col = _block(rng, 4000, 9, 9000)
    x = rng.standard_normal((9000, 96)).astype(np.float32)
    flag = torch.zeros(1, dtype=torch.int32, device=DEV)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    for swap, want in ((False, 1), (True, 0)):
        c = col.copy()
        if swap:
            c[[10, 20000]] = c[[20000, 10]]
        assert capi.lib().apt_coo_is_grouped(ctypes.c_void_p(dev(c).data_ptr()), len(c),
                                             ctypes.c_void_p(flag.data_ptr()), stream) == 0
        assert int(flag.item()) == want
        want_out = orc.spmm_sum(0, row, c, x, 4000)
        a = capi.spmm_sum(0, dev(row), dev(c), dev(x), 4000)
        b = capi.spmm_sum(0, dev(row), dev(c), dev(x), 4000, detect_grouped=False)
        assert _close(a.cpu().numpy(), want_out, 1e-5) and _close(b.cpu().numpy(), want_out, 1e-5)
        if not swap:
            assert torch.equal(a, capi.spmm_sum(0, dev(row), dev(c), dev(x), 4000))
    for n in (0, 1):                                         # nothing to compare: grouped
        assert capi.lib().apt_coo_is_grouped(ctypes.c_void_p(dev(col).data_ptr()), n,
                                             ctypes.c_void_p(flag.data_ptr()), stream) == 0
        assert int(flag.item()) == 1


@pytest.mark.parametrize("heads,hd", [(4, 64), (1, 256), (3, 8), (1, 5)])
def test_spmm_heads_owns_its_rows(orc, capi, heads, hd):
    """apt_spmm_heads with the CSR offsets of col: outputs that start as NaN come back
    complete (rows without edges zero, rows inside one wavefront range stored, rows that
    span ranges zeroed and added) and equal the oracle; weights optional."""
    rng = np.random.default_rng(heads * 31 + hd)
    rows, n_x = 5000, 900
    deg = rng.integers(0, 4, rows)
    deg[[0, 17, 4000]] = [0, 200, 70]
    deg[-3:] = 0
    indptr = np.concatenate([[0], np.cumsum(deg)])
    E = int(indptr[-1])
    col = np.repeat(np.arange(rows), deg)
    row = rng.integers(0, n_x, E)
    eids = rng.permutation(E)
    x = rng.standard_normal((n_x, heads, hd)).astype(np.float32)
    w = rng.standard_normal((E, heads)).astype(np.float32)
    w2 = rng.standard_normal((E, heads)).astype(np.float32)
    nan = lambda *shape: torch.full(shape, float("nan"), device=DEV)
    got, got2 = capi.spmm_heads(dev(row), dev(col), dev(x), dev(w), rows, weight_row=dev(eids), grouped=True,
                                head_weights2=dev(w2), out_indptr=dev(indptr), out=nan(rows, heads, hd),
                                out2=nan(rows, heads))
    want, want2 = orc.spmm_csr(indptr, row, x.reshape(n_x, -1), eids=eids, head_weights=w, head_weights2=w2,
                               heads=heads)
    assert not torch.isnan(got).any() and not torch.isnan(got2).any()
    assert _close(got.cpu().numpy().reshape(rows, -1), want, 1e-5) and _close(got2.cpu().numpy(), want2, 1e-5)
    assert not got[0].any() and not got[-1].any()
    plain = capi.spmm_heads(dev(row), dev(col), dev(x), None, rows, grouped=True, out_indptr=dev(indptr),
                            out=nan(rows, heads, hd))
    assert _close(plain.cpu().numpy().reshape(rows, -1), orc.spmm_csr(indptr, row, x.reshape(n_x, -1)), 1e-5)
    with pytest.raises(capi.AptError):
        capi.spmm_heads(dev(row), dev(col), dev(x), None, rows, grouped=False, out_indptr=dev(indptr))


def test_gat_random_shapes(orc, capi):
    """Forty random (heads, head_dim, fanout) shapes on both sides of what a wavefront
    per destination can hold (heads a power of two, heads x fanout <= 64, lanes per
    head a power of two): forward and attention weights against the oracle, fp32 and
    bf16, and empty destinations."""
    rng = np.random.default_rng(99)
    for case in range(40):
        heads = int(rng.choice([1, 2, 3, 4, 8, 16]))
        dim = int(rng.choice([4, 8, 12, 16, 32, 64, 128, 20]))
        fanout = int(rng.choice([1, 2, 3, 4, 8, 15, 16, 17, 32, 33]))
        n_dst, n_src = 700, 3000
        nbr = _ell(rng, n_dst, fanout, n_src)
        nbr.reshape(n_dst, fanout)[5] = -1                       # a destination without neighbours
        bf16 = case % 3 == 2
        ft = rng.standard_normal((n_src, heads, dim)).astype(np.float32)
        ft_t = dev(ft).to(torch.bfloat16) if bf16 else dev(ft)
        ft_ref = ft_t.float().cpu().numpy()
        el = rng.standard_normal((n_src, heads)).astype(np.float32)
        er = rng.standard_normal((n_dst, heads)).astype(np.float32)
        want, want_a = orc.gat_block(nbr, n_dst, fanout, ft_ref, el, er, 0.2, want_attn=True)
        got, got_a = capi.gat_block(dev(nbr), n_dst, fanout, ft_t, dev(el), dev(er), 0.2, want_attn=True)
        tol = 1e-2 if bf16 else 1e-5
        assert _close(got.cpu().numpy(), want, tol), (case, heads, dim, fanout, bf16)
        assert np.max(np.abs(got_a.cpu().numpy() - want_a)) <= 1e-5, (case, heads, dim, fanout)
        assert not got[5].any()


def test_gat_backward_random_shapes(capi):
    """apt_gat_block_backward against the same arithmetic written with dense torch ops on the
    fixed-stride layout (float64), for shapes on both sides of the wavefront-per-destination
    kernel's limits; fp32 and bf16 features."""
    rng = np.random.default_rng(123)
    for case in range(30):
        heads = int(rng.choice([1, 2, 3, 4, 8]))
        dim = int(rng.choice([4, 8, 16, 64, 20, 128]))
        fanout = int(rng.choice([1, 3, 8, 15, 16, 17, 33]))
        n_dst, n_src = 500, 2000
        nbr = _ell(rng, n_dst, fanout, n_src).reshape(n_dst, fanout)
        nbr[7] = -1
        bf16 = case % 3 == 2
        ft = dev(rng.standard_normal((n_src, heads, dim)).astype(np.float32))
        if bf16:
            ft = ft.to(torch.bfloat16)
        el = dev(rng.standard_normal((n_src, heads)).astype(np.float32))
        er = dev(rng.standard_normal((n_dst, heads)).astype(np.float32))
        d_out = dev(rng.standard_normal((n_dst, heads, dim)).astype(np.float32))
        nb = dev(nbr.reshape(-1))
        _, attn = capi.gat_block(nb, n_dst, fanout, ft, el, er, 0.2, want_attn=True)
        fmt = capi.block_formats(nb, n_dst, fanout, n_src, want_csr=False)
        a_edge, dz_edge, d_er = capi.gat_block_backward(nb, n_dst, fanout, ft, el, er, 0.2, attn, d_out,
                                                        fmt["csc_indptr"], fmt["num_edges"])
        # dense statement
        nbt = dev(nbr)
        valid = nbt >= 0
        idx = nbt.clamp(min=0)
        ftn = ft.double()[idx]                                                    # [n_dst, fanout, H, D]
        part = (d_out.double()[:, None] * ftn).sum(-1) * valid[..., None]         # [n_dst, fanout, H]
        a = attn.double().view(n_dst, fanout, heads)
        s = (a * part).sum(1, keepdim=True)
        z = el.double()[idx] + er.double()[:, None]
        dz = a * (part - s) * torch.where(z > 0, 1.0, 0.2) * valid[..., None]
        tol = dict(rtol=1e-4, atol=1e-4)
        assert torch.allclose(d_er.double(), dz.sum(1), **tol), (case, heads, dim, fanout, bf16)
        assert torch.allclose(a_edge.double(), a[valid], **tol), (case, heads, dim, fanout, bf16)
        assert torch.allclose(dz_edge.double(), dz[valid], **tol), (case, heads, dim, fanout, bf16)
