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
