"""Virtual-node mapping of SP mode (reference src/cuda/npc_kernel.cu:15-183):
oracle vs numpy closed forms (no GPU), HIP vs oracle, and the operators."""
import numpy as np
import pytest


def _owner(v, min_vids, world, rank, node_beg, node_end, id_offset=0):
    d = np.maximum(np.searchsorted(min_vids[1:world], v, side="right"), id_offset)
    return np.where((d < node_beg) | (d >= node_end), rank, d)


CASES = [dict(world=8, rank=3, node_beg=0, node_end=8),          # one machine
         dict(world=8, rank=5, node_beg=4, node_end=8),          # two machines: owners off this one -> rank
         dict(world=1, rank=0, node_beg=0, node_end=1),
         dict(world=4, rank=1, node_beg=0, node_end=4, id_offset=2)]


def _inputs(rng, world, num_dst=37, fanout=5):
    min_vids = np.concatenate([[0], np.sort(rng.choice(np.arange(1, 1000), world - 1, replace=False)), [1000]])
    dst = rng.integers(0, 1000, num_dst)
    src = rng.integers(0, 1000, num_dst * fanout)
    src[:world + 1] = min_vids[:world + 1].clip(max=999)        # ids on the range boundaries
    return min_vids.astype(np.int64), dst, src


def test_oracle_virtual_nodes_closed_form(orc):
    rng = np.random.default_rng(0)
    for c in CASES:
        w, fanout = c["world"], 5
        mv, dst, src = _inputs(rng, w, fanout=fanout)
        kw = dict(rank=c["rank"], node_beg=c["node_beg"], node_end=c["node_end"], id_offset=c.get("id_offset", 0))
        own = lambda v: _owner(v, mv, w, c["rank"], c["node_beg"], c["node_end"], c.get("id_offset", 0))
        nd = len(dst)
        got = orc.map_to_vir(src, fanout, mv, w, dst=dst, **kw)
        want = np.concatenate([own(dst) * nd + np.arange(nd), own(src) * nd + w * nd + np.arange(len(src)) // fanout])
        assert np.array_equal(got, want)
        got = orc.map_to_vir(src, fanout, mv, w, num_dst=nd, **kw)
        assert np.array_equal(got, own(src) * nd + np.arange(len(src)) // fanout)
        # send offsets: lower bounds of multiples of num_dst in the sorted virtual nodes / their unique values
        for with_dst in (False, True):
            vir = np.sort(orc.map_to_vir(src, fanout, mv, w, dst=dst if with_dst else None, num_dst=nd, **kw))
            uniq = np.unique(vir)
            got = orc.vir_send_offset(w, nd, vir, uniq, with_dst)
            ka = np.arange((2 if with_dst else 1) * w + 1)
            kb = np.arange(1, w + 1) + (w if with_dst else 0)
            want = np.concatenate([np.searchsorted(vir, ka * nd, "left"), np.searchsorted(uniq, kb * nd, "left")])
            assert np.array_equal(got, want)
            assert got[len(ka) - 1] == len(vir) and got[-1] == len(uniq)


@pytest.mark.gpu
def test_gpu_virtual_nodes(orc, capi):
    import torch

    import apt_amd as npc
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")
    rng = np.random.default_rng(1)
    for c in CASES:
        w, fanout = c["world"], 7
        mv, dst, src = _inputs(rng, w, num_dst=5000, fanout=fanout)
        kw = dict(rank=c["rank"], node_beg=c["node_beg"], node_end=c["node_end"], id_offset=c.get("id_offset", 0))
        for d in (dst, None):
            want = orc.map_to_vir(src, fanout, mv, w, dst=d, num_dst=len(dst), **kw)
            got = capi.map_to_vir(dev(src), fanout, dev(mv), w, dst=None if d is None else dev(d), num_dst=len(dst), **kw)
            assert np.array_equal(got.cpu().numpy(), want)
            vir = np.sort(want)
            uniq = np.unique(vir)
            got = capi.vir_send_offset(w, len(dst), dev(vir), dev(uniq), d is not None)
            assert np.array_equal(got.cpu().numpy(), orc.vir_send_offset(w, len(dst), vir, uniq, d is not None))
        # the operators read rank / world / min_vids from the registry (src/sampling.cc:19-50)
        if c.get("id_offset", 0) == 0:
            npc.set_topology(c["rank"], w, c["node_end"] - c["node_beg"])
            npc.register_min_vids(dev(mv), 0)
            got = npc.ops.srcdst_to_vir(fanout, dev(dst), dev(src))
            assert np.array_equal(got.cpu().numpy(), orc.map_to_vir(src, fanout, mv, w, dst=dst, **kw))
            got = npc.ops.src_to_vir(fanout, len(dst), dev(src))
            assert np.array_equal(got.cpu().numpy(), orc.map_to_vir(src, fanout, mv, w, num_dst=len(dst), **kw))
    npc.set_topology(0, 1)
    assert capi.map_to_vir(dev(np.empty(0, np.int64)), 3, dev(mv), 1, num_dst=0).numel() == 0


@pytest.mark.gpu
def test_spmm_operator_both_directions(orc, capi):
    """spmm_copy_u_sum over a block and over the same block with the edges reversed and the two offset
    tables swapped (how the reference forms the gradient, python/npc/model/sageconv.py:100-114), against
    torch's own index_add on the GPU in fp32."""
    import torch

    import apt_amd as npc
    rng = np.random.default_rng(2)
    n_dst, fanout, n_src, dim = 700, 6, 2500, 48
    col = torch.arange(n_dst, device="cuda:0").repeat_interleave(fanout)
    row = torch.from_numpy(rng.integers(0, n_src, n_dst * fanout)).to("cuda:0")
    coo_off = torch.tensor([0, row.numel()], device="cuda:0")
    x_off, out_off = torch.tensor([0, n_src], device="cuda:0"), torch.tensor([0, n_dst], device="cuda:0")
    x = torch.randn(n_src, dim, device="cuda:0")
    out = npc.spmm_copy_u_sum(row, col, x, coo_off, x_off, out_off)
    assert torch.allclose(out, torch.zeros(n_dst, dim, device="cuda:0").index_add(0, col, x[row]), rtol=1e-5, atol=1e-5)
    dz = torch.randn(n_dst, dim, device="cuda:0")
    dx = npc.spmm_copy_u_sum(col, row, dz, coo_off, out_off, x_off)
    assert torch.allclose(dx, torch.zeros(n_src, dim, device="cuda:0").index_add(0, row, dz[col]), rtol=1e-5, atol=1e-5)
