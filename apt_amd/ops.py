"""Python front end of the `npc` operators, with the function names and
argument order of the reference's python/npc/ops.py and python/npc/sampler.py.

Each function forwards to torch.ops.npc.<name>, registered by libnpc.so
(apt_amd/csrc/torch_bind.cc) with the schemas the reference binds in
src/pybind.cc:18-48.  The operators run on the GPU through libapt_hip.so and
have no CPU implementation; those that need other GPUs raise.
"""
from typing import Optional, Tuple

import torch

_npc = torch.ops.npc


# ---------------------------------------------------------------- registries
def cache_feats_shared(num_total_nodes: int, localnode_feats: torch.Tensor, cached_feats: torch.Tensor,
                       cached_idx: torch.Tensor, localnode_idx: Optional[torch.Tensor] = None,
                       feat_dim_offset: int = 0) -> None:
    """reference python/npc/ops.py:48-63"""
    if localnode_idx is None:
        localnode_idx = torch.arange(localnode_feats.shape[0], dtype=torch.int64)
    _npc.cache_feats_shared(num_total_nodes, localnode_feats, cached_feats, cached_idx, localnode_idx,
                            feat_dim_offset)


def mix_cache_graphs(num_cached_nodes: int, cached_node_idx: torch.Tensor, cached_indptr: torch.Tensor,
                     cached_indices: torch.Tensor, global_indptr: torch.Tensor,
                     global_indices: torch.Tensor) -> None:
    """reference python/npc/ops.py:66-81"""
    _npc.mix_cache_graphs(num_cached_nodes, cached_node_idx, cached_indptr, cached_indices,
                          global_indptr, global_indices)


def register_graph_partition(indptr, indices, row_begin: int, num_total_nodes: int) -> None:
    """Rows [row_begin, row_begin + len(indptr) - 1) live here; every other
    node has no adjacency.  No counterpart in the reference."""
    _npc.register_graph_partition(indptr, indices, row_begin, num_total_nodes)


def register_min_vids(shuffle_min_vids: torch.Tensor, shuffle_id_offset: int = 0) -> None:
    """reference python/npc/ops.py:107-110"""
    _npc.register_min_vids(shuffle_min_vids, shuffle_id_offset)


def register_multi_machines_scheme(remote_worker_map: torch.Tensor, remote_worker_id: torch.Tensor) -> None:
    """reference python/npc/ops.py:113-120 (takes the two tensors instead of args)"""
    _npc.register_multi_machines_scheme(remote_worker_map, remote_worker_id)


def set_topology(rank: int = 0, world_size: int = 1, node_size: Optional[int] = None) -> None:
    """The rank bookkeeping of npc.init (reference python/npc/__init__.py:51-58)
    without communicators: bucketing needs the rank and the number of owners."""
    _npc.set_topology(rank, world_size, node_size if node_size is not None else world_size)


def set_rng_seed(seed: int) -> None:
    _npc.set_rng_seed(seed)


def set_strict(strict: bool) -> None:
    """True (default): load_subtensor reports requested nodes that have no row here (see set_miss_check,
    "deferred"), and the pack direction of feat_shuffle checks a permutation that shuffle_seeds did not produce
    (repeated entries add up, as in the reference).  False: neither."""
    _npc.set_strict(strict)


def set_miss_check(mode: str) -> None:
    """How load_subtensor reports requested nodes without a feature row on this GPU (their rows are zero-filled;
    the reference reads out of bounds):
      "deferred" (default)  no call waits for the GPU: the miss counter follows the gather to pinned host memory
                            and the next npc operator call, or check_errors(), raises IndexError for it;
      "immediate"           load_subtensor waits for its own counter and raises itself;
      "off"                 not reported."""
    _npc.set_miss_check(mode)


def check_errors() -> None:
    """Waits for the deferred checks of earlier calls and raises IndexError if one of them failed."""
    _npc.check_errors()


def set_ranked_relabel(enabled: bool) -> None:
    """True (default): relabel_csc on a registered graph goes through the graph's rank table (and continues the
    batch when its seeds are the unique list the previous call returned); False: always the hash table."""
    _npc.set_ranked_relabel(bool(enabled))


def set_block_buffer_ring(sets: int) -> None:
    """0 (default): sample_blocks returns fresh tensors on every call, as the reference's operators do.
    n > 0: it hands out n registry-owned sets of output buffers in turn, which saves the allocations, but
    the tensors of call k are overwritten by call k + n, whoever still holds them."""
    _npc.set_block_buffer_ring(int(sets))


def block_buffer_ring() -> int:
    return int(_npc.block_buffer_ring())


# ---------------------------------------------------------------- hot path
def local_sample_one_layer(seeds: torch.Tensor, fanout: int):
    """reference python/npc/sampler.py:8-9 -> [seeds, neighbors[n * fanout]]"""
    return _npc.local_sample_one_layer(seeds, fanout)


def sample_neighbors(seeds: torch.Tensor, fanout: int, replace: bool, rng_seed: int, hop: int):
    """-> (neighbors[n * fanout] padded with -1, counts[n]); replace=False
    samples without replacement.  No counterpart in the reference."""
    return _npc.sample_neighbors(seeds, fanout, replace, rng_seed, hop)


def sample_blocks(seeds: torch.Tensor, hop_fanouts, replace: bool, rng_seed: int, formats: bool = False):
    """Every hop of a batch in one operator call (sample -> relabel -> next
    frontier; reference python/npc/sampler.py:187-203,358-364), one host wait.
    hop_fanouts: from the seeds outward.  formats: every hop's block also as
    COO + CSC, emitted before that wait.
    -> (sizes list[H + 2], input_nodes, [(neighbors, relabeled, counts) per hop])
       (+ [dict(coo_row, coo_col, csc_indptr, num_edges) per hop] with formats)"""
    H = len(hop_fanouts)
    out = _npc.sample_blocks(seeds, [int(f) for f in hop_fanouts], bool(replace), int(rng_seed), bool(formats))
    hops = [tuple(out[2 + 3 * h:5 + 3 * h]) for h in range(H)]
    sizes = out[0].tolist()
    if not formats:
        return sizes, out[1], hops
    base = 2 + 3 * H
    fmts = [dict(coo_row=out[base + 3 * h], coo_col=out[base + 3 * h + 1], csc_indptr=out[base + 3 * h + 2],
                 num_edges=sizes[H + 2 + h]) for h in range(H)]
    return sizes[:H + 2], out[1], hops, fmts


def block_formats(relabeled: torch.Tensor, num_dst: int, fanout: int, num_src: int, want_csr: bool = True):
    """COO / CSC (/ CSR) of a fixed-stride block -> dict of tensors."""
    out = _npc.block_formats(relabeled, num_dst, fanout, num_src, want_csr)
    d = dict(coo_row=out[0], coo_col=out[1], csc_indptr=out[2], num_edges=out[0].numel())
    if want_csr:
        d.update(csr_indptr=out[3], csr_indices=out[4], csr_eids=out[5])
    return d


def tensor_relabel_csc(seeds, neighbors) -> Tuple[torch.Tensor, torch.Tensor]:
    """reference python/npc/sampler.py:72-73"""
    return _npc.relabel_csc(seeds, neighbors)


relabel_csc = tensor_relabel_csc


def load_subtensor(node_id: torch.Tensor) -> torch.Tensor:
    """reference python/npc/ops.py:516-521 (single-machine branch)"""
    return _npc.load_subtensor(node_id)


def cpu_load_subtensor(node_id: torch.Tensor) -> torch.Tensor:
    return _npc.cpu_load_subtensor(node_id)


def cluster_reqs(node_id: torch.Tensor):
    return _npc.cluster_reqs(node_id)


def cluster_and_permute(seeds: torch.Tensor):
    """-> (bucket_size, bucket_offset, sorted_idx, permutation): the on-GPU half
    of shuffle_seeds for any world size."""
    return _npc.cluster_and_permute(seeds)


def shuffle_seeds(seeds: torch.Tensor):
    """reference python/npc/ops.py:603-606"""
    return _npc.shuffle_seeds(seeds)


def feat_shuffle(inputs, send_offset, recv_offset, permutation, feat_dim: int, fwd_flag: int):
    return _npc.feat_shuffle(inputs, send_offset, recv_offset, permutation, feat_dim, fwd_flag)


class NPFeatureShuffle(torch.autograd.Function):
    """reference python/npc/ops.py:633-662: forward unpacks rows by the
    permutation, backward packs the gradient back."""

    @staticmethod
    def forward(ctx, fsi, input_tensor):
        ctx.fsi = fsi
        return feat_shuffle(input_tensor, fsi.send_offset, fsi.recv_offset, fsi.permutation,
                            fsi.feat_dim, 1)

    @staticmethod
    def backward(ctx, grad_output):
        fsi = ctx.fsi
        return None, feat_shuffle(grad_output.contiguous(), fsi.recv_offset, fsi.send_offset,
                                  fsi.permutation, fsi.feat_dim, 0)


# ---------------------------------------------------------------- aggregation
def spmm_copy_u_sum(coo_row, coo_col, input, coo_offset, input_offset, output_offset):
    """reference src/spmm.cc:9-19 (python/npc/model/sageconv.py:105)"""
    return _npc.spmm_copy_u_sum(coo_row, coo_col, input, coo_offset, input_offset, output_offset)


def spmm_copy_e_sum(coo_row, coo_col, input, coo_offset, output_offset):
    return _npc.spmm_copy_e_sum(coo_row, coo_col, input, coo_offset, output_offset)


def spmm_u_mul_e_sum(coo_row, coo_col, input, edata, coo_offset, input_offset, output_offset):
    return _npc.spmm_u_mul_e_sum(coo_row, coo_col, input, edata, coo_offset, input_offset, output_offset)


def sddmm_u_add_v(coo_row, coo_col, lhs, rhs, coo_offset, lhs_offset, rhs_offset):
    return _npc.sddmm_u_add_v(coo_row, coo_col, lhs, rhs, coo_offset, lhs_offset, rhs_offset)


def sddmm_u_mul_v(coo_row, coo_col, lhs, rhs, coo_offset, lhs_offset, rhs_offset):
    return _npc.sddmm_u_mul_v(coo_row, coo_col, lhs, rhs, coo_offset, lhs_offset, rhs_offset)


def srcdst_to_vir(fanout: int, dst: torch.Tensor, src: torch.Tensor) -> torch.Tensor:
    """reference python/npc/sampler.py:20-21"""
    return _npc.srcdst_to_vir(fanout, dst, src)


def src_to_vir(fanout: int, num_dst: int, src: torch.Tensor) -> torch.Tensor:
    """reference python/npc/sampler.py:16-17"""
    return _npc.src_to_vir(fanout, num_dst, src)


def np_sample_and_shuffle(seeds, fanout):
    return _npc.np_sample_and_shuffle(seeds, fanout)
