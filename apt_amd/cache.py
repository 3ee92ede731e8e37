"""Choosing and building the GPU caches: the callers either side of the
registries (reference python/npc/ops.py:107-274 cache_adj_and_feats,
:304-497 load_partition, examples/dryrun.py:86-108 access counting).

The reference's policies read per-rank files written by earlier runs and then
do tensor arithmetic on them.  The arithmetic is kept, policy by policy, on
in-memory tensors (the caller loads the files: save_hotness / load_hotness use
the reference's format); cache construction, one Python slice per node in the
reference, runs on the GPU on device-resident arrays.
"""
from collections import namedtuple

import torch

from . import capi, ops

BYTES_PER_ELEMENT = 4  # python/npc/ops.py:20: budgets are counted in fp32 elements

# python/npc/ops.py:23-32
PartData = namedtuple("PartData", ["min_vids", "train_nid", "labels", "cache_mask", "num_cached_feat_nodes",
                                   "num_cached_feat_elements", "num_cached_graph_nodes",
                                   "num_cached_graph_elements"])


# --------------------------------------------------------------------------
# dry run: access counting
# --------------------------------------------------------------------------
class HotnessCounter:
    """The two access counters of a dry run (examples/dryrun.py:86-92):
    counter[0] over the batch's output nodes (seeds), counter[1] over its input
    nodes; add_* after every batch."""

    def __init__(self, num_total_nodes, device="cuda:0"):
        self.dst_count = torch.zeros(num_total_nodes, dtype=torch.int64, device=device)
        self.src_count = torch.zeros(num_total_nodes, dtype=torch.int64, device=device)

    @property
    def freq(self):
        """Input-node frequencies, the list entry every policy reads (ops.py:188)."""
        return self.src_count

    def add(self, input_nodes, n_dev=None, output_nodes=None):
        """input_nodes: node ids a batch reads features of (device int64); n_dev:
        optional device-side count, so the pipeline's node list can be counted
        without a host sync."""
        capi.count_ids(input_nodes, self.src_count, n_dev=n_dev)
        if output_nodes is not None:
            capi.count_ids(output_nodes, self.dst_count)

    def save(self, path):
        save_hotness(path, self.dst_count, self.src_count)


def save_hotness(path, dst_count, src_count):
    """The reference's file: torch.save of the list [dst_count, src_count] of
    int64 CPU tensors (examples/dryrun.py:86,108)."""
    torch.save([dst_count.cpu(), src_count.cpu()], path)


def load_hotness(path, device="cpu"):
    """-> [dst_count, src_count]; plain tensors only are accepted."""
    dst, src = torch.load(path, weights_only=True, map_location=device)
    return [dst, src]


# --------------------------------------------------------------------------
# policies (python/npc/ops.py:107-274); every one returns
# (cache_feat_node_idx, cache_graph_node_idx)
# --------------------------------------------------------------------------
def rank_by_hotness(freq, candidates=None):
    """Node ids by decreasing frequency (ops.py:188,213); ties keep id order
    (torch.sort there leaves tie order open).  `candidates`: optional bool mask,
    ids outside it are dropped (ops.py:243-245)."""
    order = torch.sort(freq, descending=True, stable=True).indices
    if candidates is not None:
        order = order[candidates[order]]
    return order


def local_mask(localnode_feats_idx, num_total_nodes):
    mask = torch.zeros(num_total_nodes, dtype=torch.bool, device=localnode_feats_idx.device)
    mask[localnode_feats_idx] = True
    return mask


def policy_dryrun(freq, localnode_feats_idx, num_total_nodes, cache_memory, input_dim, base=1):
    """"dryrun" mode (ops.py:170-260): no graph cache; features of the most
    frequently read nodes that have a local row, as many as
    cache_memory*base / (input_dim*4) (base = world size under MP, where every
    rank caches a column slice)."""
    ranked = rank_by_hotness(freq, local_mask(localnode_feats_idx, num_total_nodes))
    n = min(ranked.numel(), int(cache_memory * base / (input_dim * BYTES_PER_ELEMENT)))
    return ranked[:n].contiguous(), ranked.new_empty(0)


def policy_costmodel(sorted_idx, idx_mem, num_total_nodes, cache_memory):
    """"costmodel" mode (ops.py:119-141).  sorted_idx ranks entries of a joint
    id space: id < N is node id's feature row, id >= N the adjacency row of node
    id-N; idx_mem[id] is the bytes either takes.  The prefix kept is the
    reference's: (first position whose running total exceeds the budget) - 1,
    and nothing when the total never exceeds it (torch.max of an all-False
    mask returns position 0)."""
    over = torch.cumsum(idx_mem[sorted_idx], 0) > cache_memory
    first = int(torch.nonzero(over)[0].item()) if bool(over.any()) else 0
    keep = sorted_idx[:max(0, first - 1)]
    return keep[keep < num_total_nodes].contiguous(), (keep[keep >= num_total_nodes] - num_total_nodes).contiguous()


def policy_greedy(feat_idx, graph_idx, idx_mem, num_total_nodes, cache_memory, feat_ratio):
    """"greedy" mode (ops.py:143-169): the largest m (binary search over
    [0, N)) such that the first m*ratio ranked feature rows plus the first
    m*(1-ratio) ranked adjacency rows fit the budget.  As in the reference the
    running totals are read at position k for "k entries", i.e. one entry more
    than is then cached."""
    feat_mem = torch.cumsum(idx_mem[feat_idx], 0)
    graph_mem = torch.cumsum(idx_mem[graph_idx + num_total_nodes], 0)
    lb, ub = 0, num_total_nodes
    while ub > lb + 1:
        mid = (ub + lb) // 2
        total = (feat_mem[int(mid * feat_ratio)] + graph_mem[int(mid * (1 - feat_ratio))]).item()
        if total <= cache_memory:
            lb = mid
        else:
            ub = mid
    return (feat_idx[:int(lb * feat_ratio)].contiguous(), graph_idx[:int(lb * (1 - feat_ratio))].contiguous())


def policy_random(localnode_feats_idx, feat_cache_ratio, generator=None):
    """Fallback mode (ops.py:262-273): a random feat_cache_ratio of the local
    rows, no graph cache."""
    n_local = localnode_feats_idx.numel()
    n = int(feat_cache_ratio * n_local)
    pick = torch.randperm(n_local, generator=generator, device=localnode_feats_idx.device)[:n]
    return localnode_feats_idx[pick].contiguous(), localnode_feats_idx.new_empty(0)


def policy_graph_by_budget(graph, ranked_ids, memory_bytes):
    """Longest prefix of ranked_ids whose CSR (8 bytes per offset and per edge)
    fits the budget.  Not a reference mode: the graph-side counterpart of
    policy_dryrun, for a single GPU that caches adjacency by measured hotness."""
    if ranked_ids.numel() == 0 or memory_bytes <= 0:
        return ranked_ids[:0]
    deg = capi.csr_row_degrees(graph, ranked_ids)
    used = torch.cumsum((deg + 1) * 8, 0)
    return ranked_ids[:int((used <= memory_bytes).sum().item())].contiguous()


# --------------------------------------------------------------------------
# construction + registration (python/npc/ops.py:304-497)
# --------------------------------------------------------------------------
def build_graph_cache(graph, node_ids):
    """-> (cached_indptr, cached_indices) of node_ids' adjacency rows
    (ops.py:370-384)."""
    return capi.csr_select_rows(graph, node_ids)


def build_feature_cache(localnode_feats, localnode_feats_idx, num_total_nodes, node_ids, col_begin=0, col_end=None):
    """-> localnode_feats[row of node_ids, col_begin:col_end] (ops.py:405-437);
    every id must have a local row."""
    dev = localnode_feats.device
    col_end = localnode_feats.shape[1] if col_end is None else col_end
    pos = torch.full((num_total_nodes,), -1, dtype=torch.int64, device=dev)
    pos[localnode_feats_idx] = -torch.arange(localnode_feats_idx.numel(), dtype=torch.int64, device=dev) - 2
    store = capi.FeatStore(localnode_feats, None, pos, col_offset=col_begin, out_dim=col_end - col_begin,
                           num_total_nodes=num_total_nodes)
    if node_ids.numel() == 0:
        return localnode_feats.new_empty((0, col_end - col_begin))
    miss = torch.zeros(1, dtype=torch.int64, device=dev)
    out = capi.gather_rows(store, node_ids, miss_count=miss)
    if int(miss.item()):
        raise IndexError("build_feature_cache: %d ids have no local feature row" % int(miss.item()))
    return out


def load_partition(rank, min_vids, localnode_feats_idx, localnode_feats, labels, train_mask, indptr, indices,
                   cache_feat_node_idx, cache_graph_node_idx, max_cache_feat_nodes=-1, max_cache_graph_nodes=-1,
                   feat_dim_begin=0, feat_dim_end=None, row_begin=0):
    """In-memory, one-GPU counterpart of load_partition (ops.py:304-497): applies
    the forced limits, builds both caches on the GPU, registers graph, features
    and min_vids with the operators and returns the reference's PartData.

    All tensors live on the GPU.  (feat_dim_begin, feat_dim_end): the column
    slice this rank caches under MP (ops.py:414-420), whole rows otherwise.
    row_begin: first node of a contiguous-range adjacency partition."""
    dev = indptr.device
    num_total_nodes = int(min_vids[-1])
    if 0 <= max_cache_feat_nodes < cache_feat_node_idx.numel():
        cache_feat_node_idx = cache_feat_node_idx[:max_cache_feat_nodes]
    if 0 <= max_cache_graph_nodes < cache_graph_node_idx.numel():
        cache_graph_node_idx = cache_graph_node_idx[:max_cache_graph_nodes]
    cache_feat_node_idx = cache_feat_node_idx.to(dev).contiguous()
    cache_graph_node_idx = cache_graph_node_idx.to(dev).contiguous()
    # graph cache
    graph = capi.Graph(indptr, indices, row_begin=row_begin, num_total_nodes=num_total_nodes)
    c_indptr, c_indices = build_graph_cache(graph, cache_graph_node_idx)
    if row_begin:
        if cache_graph_node_idx.numel():
            raise ValueError("a graph cache on top of a range partition is not supported")
        ops.register_graph_partition(indptr, indices, row_begin, num_total_nodes)
    else:
        ops.mix_cache_graphs(cache_graph_node_idx.numel(), cache_graph_node_idx, c_indptr, c_indices, indptr, indices)
    # feature cache
    cached = build_feature_cache(localnode_feats, localnode_feats_idx, num_total_nodes, cache_feat_node_idx,
                                 feat_dim_begin, feat_dim_end)
    ops.cache_feats_shared(num_total_nodes, localnode_feats, cached, cache_feat_node_idx, localnode_feats_idx,
                           feat_dim_begin)
    # training nodes of this rank, labels, cache mask
    lo, hi = int(min_vids[rank]), int(min_vids[rank + 1])
    train_nid = torch.nonzero(train_mask[lo:hi]).flatten().to(dev) + lo
    cache_mask = torch.zeros(num_total_nodes, dtype=torch.bool, device=dev)
    cache_mask[cache_feat_node_idx] = True
    mv = torch.as_tensor(list(map(int, min_vids)), dtype=torch.int64, device=dev)
    ops.register_min_vids(mv)
    return PartData(mv, train_nid, labels.to(dev), cache_mask, cache_feat_node_idx.numel(),
                    cache_feat_node_idx.numel() * cached.shape[1], cache_graph_node_idx.numel(), c_indices.numel())
