"""Writes tests/golden/minibatch_small.npz: one small, fully specified mini-batch
(graph, seeds, rng key) with the outputs of the CPU oracle.

The reference holds no fixture for this path (its tests cover NCCL collectives
only), so these vectors do not come from it: they freeze the behaviour of this
build's oracle after it was pinned by known-answer vectors and closed forms,
so that a later change to the RNG keying, the Floyd order or the relabel order
shows up as a diff against committed data.  Run from the repository root:

    python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import oracle as orc  # noqa: E402
from apt_amd.synth import rmat_csr_numpy  # noqa: E402


def main():
    n = 300
    indptr, indices = rmat_csr_numpy(n, 3000, seed=17)
    rng = np.random.default_rng(18)
    seeds = rng.permutation(n)[:24]
    seeds[5] = seeds[2]                                   # a repeated seed
    g = orc.Graph(indptr, indices)
    out = dict(indptr=indptr, indices=indices, seeds=seeds, hops=np.array([3, 4]), rng_seed=np.array([20240229]))
    for tag, replace in (("norep", False), ("rep", True)):
        inp, blocks = orc.sample_blocks(g, seeds, [3, 4], replace, 20240229)
        if not replace:
            blocks_norep = blocks
        out[f"{tag}_input_nodes"] = inp
        for h, b in enumerate(reversed(blocks)):
            out[f"{tag}_hop{h}_neighbors"] = b["neighbors"]
            out[f"{tag}_hop{h}_counts"] = b["counts"]
            out[f"{tag}_hop{h}_relabeled"] = b["relabeled"]
    feats = rng.standard_normal((n, 6)).astype(np.float32)
    out["feats"] = feats
    out["norep_features"] = orc.gather_rows(orc.FeatStore(feats), out["norep_input_nodes"])[0]
    min_vids = np.array([0, 70, 150, 220, 300])
    bs, bo, so, pm = orc.cluster_permute(out["norep_input_nodes"], min_vids, 4, 0, 1, 0, 4)
    out.update(min_vids=min_vids, bucket_size=bs, bucket_offset=bo, bucket_sorted=so, bucket_perm=pm)
    # the callers either side of the core path, on the same batch
    blk = blocks_norep[0]                                  # outermost block
    nd, ns, fo = len(blk["seeds"]), len(blk["unique"]), int(blk["fanout"])
    fmt = orc.block_formats(blk["relabeled"], nd, fo, ns)
    for k in ("coo_row", "coo_col", "csc_indptr", "csr_indptr", "csr_indices", "csr_eids"):
        out["fmt_" + k] = fmt[k]
    out["vir_srcdst"] = orc.map_to_vir(blk["neighbors"].clip(min=0), fo, min_vids, 4, rank=1, dst=blk["seeds"])
    out["vir_src"] = orc.map_to_vir(blk["neighbors"].clip(min=0), fo, min_vids, 4, rank=1, num_dst=nd)
    vs = np.sort(out["vir_src"])
    out["vir_send_offset"] = orc.vir_send_offset(4, nd, vs, np.unique(vs), False)
    freq = np.zeros(n, dtype=np.int64)
    orc.count_ids(out["norep_input_nodes"], freq)
    orc.count_ids(out["rep_input_nodes"], freq)
    out["freq"] = freq
    hot = np.argsort(-freq, kind="stable")[:40]
    out["hot"] = hot
    out["hot_indptr"], out["hot_indices"] = orc.csr_select_rows(g, hot)
    ft = rng.standard_normal((ns, 2, 4)).astype(np.float32)
    attn = rng.standard_normal((2, 2, 4)).astype(np.float32)
    el, er = orc.gat_scores(ft, attn[0]), orc.gat_scores(ft[:nd], attn[1])
    gat, gat_a = orc.gat_block(blk["relabeled"], nd, fo, ft, el, er, 0.2, want_attn=True)
    out.update(gat_ft=ft, gat_attn=attn, gat_el=el, gat_er=er, gat_out=gat, gat_weights=gat_a)
    np.savez_compressed(os.path.join(os.path.dirname(os.path.abspath(__file__)), "minibatch_small.npz"), **out)
    print("wrote minibatch_small.npz:", {k: v.shape for k, v in out.items()})


if __name__ == "__main__":
    main()
