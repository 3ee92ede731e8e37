"""Committed vectors (tests/golden/minibatch_small.npz, written by
tests/golden/make_fixtures.py): the oracle on the CPU and the HIP library on the
GPU must both reproduce them bit for bit."""
import os

import numpy as np
import pytest

FIX = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "minibatch_small.npz")


def _load():
    return np.load(FIX, allow_pickle=False)


def test_oracle_reproduces_golden(orc):
    z = _load()
    g = orc.Graph(z["indptr"], z["indices"])
    hops = z["hops"].tolist()
    for tag, replace in (("norep", False), ("rep", True)):
        inp, blocks = orc.sample_blocks(g, z["seeds"], hops, replace, int(z["rng_seed"][0]))
        assert np.array_equal(inp, z[f"{tag}_input_nodes"])
        for h, b in enumerate(reversed(blocks)):
            for k in ("neighbors", "counts", "relabeled"):
                assert np.array_equal(b[k], z[f"{tag}_hop{h}_{k}"]), (tag, h, k)
    assert np.array_equal(orc.gather_rows(orc.FeatStore(z["feats"]), z["norep_input_nodes"])[0],
                          z["norep_features"])
    got = orc.cluster_permute(z["norep_input_nodes"], z["min_vids"], 4, 0, 1, 0, 4)
    for a, k in zip(got, ("bucket_size", "bucket_offset", "bucket_sorted", "bucket_perm")):
        assert np.array_equal(a, z[k])


def _outer_block(z):
    """Sizes of the outermost block of the no-replacement batch: (num_dst, num_src, fanout)."""
    hops = z["hops"].tolist()
    rel = z[f"norep_hop{len(hops) - 1}_relabeled"]
    return len(rel) // hops[-1], len(z["norep_input_nodes"]), hops[-1]


def test_oracle_reproduces_golden_callers(orc):
    z = _load()
    nd, ns, fo = _outer_block(z)
    rel, nbr = z["norep_hop1_relabeled"], z["norep_hop1_neighbors"]
    fmt = orc.block_formats(rel, nd, fo, ns)
    for k in ("coo_row", "coo_col", "csc_indptr", "csr_indptr", "csr_indices", "csr_eids"):
        assert np.array_equal(fmt[k], z["fmt_" + k]), k
    front = z["norep_input_nodes"][:nd]                    # the block's seeds: the node list after the first hop
    assert np.array_equal(orc.map_to_vir(nbr.clip(min=0), fo, z["min_vids"], 4, rank=1, dst=front), z["vir_srcdst"])
    assert np.array_equal(orc.map_to_vir(nbr.clip(min=0), fo, z["min_vids"], 4, rank=1, num_dst=nd), z["vir_src"])
    vs = np.sort(z["vir_src"])
    assert np.array_equal(orc.vir_send_offset(4, nd, vs, np.unique(vs), False), z["vir_send_offset"])
    freq = np.zeros(len(z["indptr"]) - 1, dtype=np.int64)
    orc.count_ids(z["norep_input_nodes"], freq)
    orc.count_ids(z["rep_input_nodes"], freq)
    assert np.array_equal(freq, z["freq"])
    ip, ix = orc.csr_select_rows(orc.Graph(z["indptr"], z["indices"]), z["hot"])
    assert np.array_equal(ip, z["hot_indptr"]) and np.array_equal(ix, z["hot_indices"])
    el, er = orc.gat_scores(z["gat_ft"], z["gat_attn"][0]), orc.gat_scores(z["gat_ft"][:nd], z["gat_attn"][1])
    assert np.array_equal(el, z["gat_el"]) and np.array_equal(er, z["gat_er"])
    out, a = orc.gat_block(rel, nd, fo, z["gat_ft"], el, er, 0.2, want_attn=True)
    assert np.array_equal(out, z["gat_out"]) and np.array_equal(a, z["gat_weights"])


@pytest.mark.gpu
def test_gpu_reproduces_golden_callers(capi):
    import torch
    z = _load()
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")
    nd, ns, fo = _outer_block(z)
    rel, nbr = z["norep_hop1_relabeled"], z["norep_hop1_neighbors"]
    fmt = capi.block_formats(dev(rel), nd, fo, ns)
    for k in ("coo_row", "coo_col", "csc_indptr", "csr_indptr", "csr_indices", "csr_eids"):
        assert np.array_equal(fmt[k].cpu().numpy(), z["fmt_" + k]), k
    got = capi.map_to_vir(dev(nbr.clip(min=0)), fo, dev(z["min_vids"]), 4, rank=1, num_dst=nd)
    assert np.array_equal(got.cpu().numpy(), z["vir_src"])
    got = capi.map_to_vir(dev(nbr.clip(min=0)), fo, dev(z["min_vids"]), 4, rank=1, dst=dev(z["norep_input_nodes"][:nd]))
    assert np.array_equal(got.cpu().numpy(), z["vir_srcdst"])
    vs = np.sort(z["vir_src"])
    got = capi.vir_send_offset(4, nd, dev(vs), dev(np.unique(vs)), False)
    assert np.array_equal(got.cpu().numpy(), z["vir_send_offset"])
    freq = torch.zeros(len(z["indptr"]) - 1, dtype=torch.int64, device="cuda:0")
    capi.count_ids(dev(z["norep_input_nodes"]), freq)
    capi.count_ids(dev(z["rep_input_nodes"]), freq)
    assert np.array_equal(freq.cpu().numpy(), z["freq"])
    ip, ix = capi.csr_select_rows(capi.Graph(dev(z["indptr"]), dev(z["indices"])), dev(z["hot"]))
    assert np.array_equal(ip.cpu().numpy(), z["hot_indptr"]) and np.array_equal(ix.cpu().numpy(), z["hot_indices"])
    ft = dev(z["gat_ft"])
    el, er = capi.gat_scores(ft, dev(z["gat_attn"][0])), capi.gat_scores(ft[:nd].contiguous(), dev(z["gat_attn"][1]))
    assert np.allclose(el.cpu().numpy(), z["gat_el"], rtol=1e-5, atol=1e-6)
    out, a = capi.gat_block(dev(rel), nd, fo, ft, dev(z["gat_el"]), dev(z["gat_er"]), 0.2, want_attn=True)
    assert np.allclose(out.cpu().numpy(), z["gat_out"], rtol=1e-5, atol=1e-6)       # fp32 vs the double-accumulating oracle
    assert np.allclose(a.cpu().numpy(), z["gat_weights"], rtol=1e-5, atol=1e-6)


@pytest.mark.gpu
def test_gpu_reproduces_golden(capi):
    import torch
    from apt_amd.pipeline import MiniBatchPipeline
    z = _load()
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")
    g = capi.Graph(dev(z["indptr"]), dev(z["indices"]))
    fs = capi.FeatStore(dev(z["feats"]))
    hops = z["hops"].tolist()
    for tag, replace in (("norep", False), ("rep", True)):
        for fused in (True, False):
            pipe = MiniBatchPipeline(g, fs, len(z["seeds"]), hops, replace=replace, fused=fused)
            pipe.run(dev(z["seeds"]), int(z["rng_seed"][0]))
            res = pipe.result()
            assert np.array_equal(res["input_nodes"].cpu().numpy(), z[f"{tag}_input_nodes"])
            for h, b in enumerate(reversed(res["blocks"])):
                for k in ("neighbors", "counts", "relabeled"):
                    assert np.array_equal(b[k].cpu().numpy(), z[f"{tag}_hop{h}_{k}"]), (tag, fused, h, k)
            if tag == "norep":
                assert np.array_equal(res["features"].cpu().numpy(), z["norep_features"])
    got = capi.cluster_permute(dev(z["norep_input_nodes"]), dev(z["min_vids"]), 4, 0, 1, 0, 4)
    for a, k in zip(got, ("bucket_size", "bucket_offset", "bucket_sorted", "bucket_perm")):
        assert np.array_equal(a.cpu().numpy(), z[k])
