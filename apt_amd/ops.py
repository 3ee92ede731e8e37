"""The operators of the mini-batch construction path, with the names, argument
order and return values the reference binds in src/pybind.cc:18-48.

Every operator runs on the GPU through the C ABI (apt_amd/capi.py); there is no
CPU implementation behind them.  Operators whose reference implementation
talks to other GPUs over NCCL are not provided; asking for them raises.
"""
import torch

from . import capi
from .state import state

ENCODE_ID = lambda i: -i - 2   # reference src/utils.h:17
FEAT_NOT_EXIST = -1            # reference src/utils.h:20


def _device():
    if not torch.cuda.is_available():
        raise RuntimeError("apt_amd needs a GPU: the operators have no CPU implementation")
    return torch.device("cuda", torch.cuda.current_device())


def _ids(t, name, dev=None):
    if not isinstance(t, torch.Tensor) or t.dtype != torch.int64:
        raise TypeError(f"{name} must be an int64 tensor")
    if t.dim() != 1:
        raise ValueError(f"{name} must be 1-D")
    if dev is not None:
        t = t.to(dev)
    return t.contiguous()


def set_topology(rank=0, world_size=1, node_size=None, local_rank=None):
    """Stands in for the rank bookkeeping of Initialize (reference
    src/core.cc:54-100) without creating communicators: bucketing needs to know
    which rank it is and how many owners there are."""
    st = state()
    st.rank, st.world_size = int(rank), int(world_size)
    st.node_size = int(node_size if node_size is not None else world_size)
    st.local_rank = int(local_rank if local_rank is not None else rank % max(st.node_size, 1))


def set_rng_seed(seed):
    st = state()
    st.rng_seed, st.sample_calls = int(seed), 0


# ---------------------------------------------------------------- registries
def cache_feats_shared(num_total_nodes, localnode_feats, cached_feats, cached_idx,
                       localnode_idx=None, feat_dim_offset=0):
    """Registers the feature tables (reference src/cache_feats.cc:14-61).

    feat_pos_map[v] = row of cached_feats if v is cached, else ENCODE_ID(row of
    localnode_feats) if v is local, else -1; the cache wins (:49-55).  Both
    tables live in HBM here (the reference keeps the local table in pinned
    host memory); a CPU tensor is copied to the GPU once.
    """
    dev = _device()
    st = state()
    if localnode_feats.dim() != 2:
        raise ValueError("localnode_feats must be [num_local, feat_dim]")
    n_local, feat_dim = localnode_feats.shape
    local = localnode_feats.to(dev).contiguous()
    if localnode_idx is None:
        localnode_idx = torch.arange(n_local, dtype=torch.int64)
    localnode_idx = _ids(localnode_idx, "localnode_idx", dev)
    cached_idx = _ids(cached_idx, "cached_idx", dev)
    if localnode_idx.numel() != n_local:
        raise ValueError("localnode_idx must name every row of localnode_feats")
    n_cached = cached_feats.shape[0] if cached_feats is not None and cached_feats.dim() == 2 else 0
    if cached_idx.numel() != n_cached:
        raise ValueError("cached_idx must name every row of cached_feats")
    for name, t in (("localnode_idx", localnode_idx), ("cached_idx", cached_idx)):
        if t.numel() and (int(t.min()) < 0 or int(t.max()) >= num_total_nodes):
            raise ValueError(f"{name} holds ids outside [0, {num_total_nodes})")
    rank_dim = cached_feats.shape[1] if n_cached else feat_dim - int(feat_dim_offset)
    if feat_dim_offset < 0 or feat_dim_offset + rank_dim > feat_dim:
        raise ValueError("feat_dim_offset + cached width exceeds the local feature width")
    pos = torch.full((num_total_nodes,), FEAT_NOT_EXIST, dtype=torch.int64, device=dev)
    pos[localnode_idx] = ENCODE_ID(torch.arange(n_local, dtype=torch.int64, device=dev))
    st.cpu_feat_pos_map = pos.cpu()
    cache = None
    if n_cached:
        cache = cached_feats.to(dev).contiguous()
        pos[cached_idx] = torch.arange(n_cached, dtype=torch.int64, device=dev)
    identity = (n_cached == 0 and n_local == num_total_nodes and
                bool(torch.equal(localnode_idx, torch.arange(n_local, dtype=torch.int64, device=dev))))
    st.local_feats = local
    st.feat_pos_map = pos
    st.feat = capi.FeatStore(local, cache, None if identity else pos, col_offset=int(feat_dim_offset),
                             out_dim=int(rank_dim), num_total_nodes=int(num_total_nodes))


def mix_cache_graphs(num_cached_nodes, cached_node_idx, cached_indptr, cached_indices,
                     global_indptr, global_indices):
    """Registers the graph tables (reference src/cache_graphs.cc:12-49):
    adj_pos_map[v] = cache row if v is cached else ENCODE_ID(v)."""
    dev = _device()
    cached_node_idx = _ids(cached_node_idx, "cached_node_idx", dev)
    if num_cached_nodes != cached_node_idx.numel():
        raise ValueError("num_cached_nodes != cached_node_idx.numel()")   # reference CHECK :19
    g_indptr = _ids(global_indptr, "global_indptr", dev)
    g_indices = _ids(global_indices, "global_indices", dev)
    total = g_indptr.numel() - 1
    if total < 0:
        raise ValueError("global_indptr is empty")
    if num_cached_nodes == 0:
        state().graph = capi.Graph(g_indptr, g_indices)
        return
    c_indptr = _ids(cached_indptr, "cached_indptr", dev)
    c_indices = _ids(cached_indices, "cached_indices", dev)
    if c_indptr.numel() != num_cached_nodes + 1:
        raise ValueError("cached_indptr must have num_cached_nodes + 1 entries")
    if int(cached_node_idx.min()) < 0 or int(cached_node_idx.max()) >= total:
        raise ValueError("cached_node_idx holds ids outside the graph")
    pos = ENCODE_ID(torch.arange(total, dtype=torch.int64, device=dev))
    pos[cached_node_idx] = torch.arange(num_cached_nodes, dtype=torch.int64, device=dev)
    state().graph = capi.Graph(g_indptr, g_indices, cached_indptr=c_indptr, cached_indices=c_indices,
                               adj_pos_map=pos)


def register_graph_partition(indptr, indices, row_begin, num_total_nodes):
    """A contiguous-range partition: rows [row_begin, row_begin + len(indptr)-1)
    are here, every other node has no adjacency (degree 0).  No counterpart in
    the reference, which always holds the whole graph in host memory."""
    dev = _device()
    state().graph = capi.Graph(_ids(indptr, "indptr", dev), _ids(indices, "indices", dev),
                               row_begin=int(row_begin), num_total_nodes=int(num_total_nodes))


def register_min_vids(shuffle_min_vids, shuffle_id_offset=0):
    """reference src/core.cc:102-108"""
    st = state()
    st.shuffle_min_vids = _ids(shuffle_min_vids, "shuffle_min_vids", _device())
    st.shuffle_id_offset = int(shuffle_id_offset)


def register_multi_machines_scheme(remote_worker_map, remote_worker_id):
    """reference src/core.cc:110-125 (state only; no communicator)"""
    st = state()
    st.remote_worker_map = _ids(remote_worker_map, "remote_worker_map", _device())
    st.remote_worker_id = [int(x) for x in remote_worker_id.tolist()]
    st.num_remote_workers = len(st.remote_worker_id)


# ---------------------------------------------------------------- hot path
def _graph():
    g = state().graph
    if g is None:
        raise RuntimeError("no graph registered: call mix_cache_graphs first")
    return g


def sample_neighbors(seeds, fanout, replace, rng_seed, hop):
    """One hop of uniform sampling -> (neighbors [n*fanout] padded with -1,
    counts [n]).  replace=False is sampling without replacement
    (count = min(fanout, degree)); no counterpart in the reference."""
    g = _graph()
    return capi.sample_neighbors(g, _ids(seeds, "seeds", g.device), int(fanout), bool(replace),
                                 int(rng_seed), int(hop))


def local_sample_one_layer(seeds, fanout):
    """reference src/sampling.cc:13-17 -> [seeds, neighbors[n*fanout]]: fanout
    draws with replacement per seed.  Unlike the reference, whose generator is
    re-seeded with the same constant on every call (src/cuda/npc_kernel.cu:258-261,292),
    successive calls use successive counter words, and rows without neighbours
    are filled with -1 instead of being left uninitialised."""
    st = state()
    g = _graph()
    s = _ids(seeds, "seeds", g.device)
    nbrs, _ = capi.sample_neighbors(g, s, int(fanout), True, st.rng_seed, st.sample_calls,
                                    want_counts=False)
    st.sample_calls += 1
    return [s, nbrs]


def relabel_csc(seeds, neighbors):
    """reference src/relabel.cc:9-15 -> [unique, relabeled]"""
    dev = _device()
    u, r, _ = capi.relabel(_ids(seeds, "seeds", dev), _ids(neighbors, "neighbors", dev))
    return [u, r]


def load_subtensor(node_id):
    """reference src/load_subtensor.cc:19-40 -> features [n, rank_feat_dim]"""
    st = state()
    if st.feat is None:
        raise RuntimeError("no features registered: call cache_feats_shared first")
    idx = _ids(node_id, "node_id", st.feat.device)
    if not st.strict:
        return capi.gather_rows(st.feat, idx)
    miss = torch.zeros(1, dtype=torch.int64, device=idx.device)
    out = capi.gather_rows(st.feat, idx, miss_count=miss)
    m = int(miss.item())
    if m:
        raise IndexError(f"load_subtensor: {m} requested node(s) have no feature row on this GPU")
    return out


def cpu_load_subtensor(node_id):
    """reference src/load_subtensor.cc:10-17: two index_selects through the
    cache-free position map (torch's own operators, as in the reference)."""
    st = state()
    if st.cpu_feat_pos_map is None:
        raise RuntimeError("no features registered: call cache_feats_shared first")
    pos = ENCODE_ID(st.cpu_feat_pos_map.index_select(0, node_id.cpu()))
    return st.local_feats.index_select(0, pos.to(st.local_feats.device))


def cluster_and_permute(seeds):
    """The on-GPU half of ShuffleSeeds (reference src/sampling.cc:159-175,
    src/cuda/npc_kernel.cu:434-470) -> (bucket_size, bucket_offset, sorted_idx,
    permutation) for any world size."""
    st = state()
    if st.shuffle_min_vids is None:
        raise RuntimeError("register_min_vids has not been called")
    node_beg = st.rank - (st.rank % st.node_size)
    return capi.cluster_permute(_ids(seeds, "seeds", _device()), st.shuffle_min_vids, st.world_size,
                                st.shuffle_id_offset, st.rank, node_beg, node_beg + st.node_size)


def shuffle_seeds(seeds):
    """reference src/sampling.cc:159-193 -> (recv_frontier, permutation,
    recv_offset, dev_offset).  With one GPU the two all-to-alls are identity
    copies; with more the exchange needs peers and is not provided."""
    st = state()
    if st.world_size != 1:
        raise NotImplementedError("shuffle_seeds exchanges ids between GPUs; only world_size 1 is "
                                  "available here (cluster_and_permute gives the local half)")
    size, offset, sorted_idx, perm = cluster_and_permute(seeds)
    off = offset.cpu()
    return sorted_idx, perm, off.clone(), off


def cluster_reqs(node_id):
    """reference src/load_subtensor.cc:83-86 -> (bucket_size, sorted_idx, permutation)"""
    st = state()
    if st.feat_pos_map is None or st.remote_worker_map is None or st.shuffle_min_vids is None:
        raise RuntimeError("cluster_reqs needs cache_feats_shared, register_min_vids and "
                           "register_multi_machines_scheme")
    size, _, sorted_idx, perm = capi.cluster_reqs(
        _ids(node_id, "node_id", _device()), st.feat_pos_map, st.remote_worker_map,
        st.shuffle_min_vids, st.world_size, st.num_remote_workers)
    return size, sorted_idx, perm


def feat_shuffle(inputs, send_offset, recv_offset, permutation, feat_dim, fwd_flag):
    """reference src/feat_shuffle.cc:9-30 with one GPU (the all-to-all is an
    identity copy): forward = rows gathered by permutation, backward = rows
    scattered to permutation."""
    st = state()
    if st.world_size != 1:
        raise NotImplementedError("feat_shuffle exchanges rows between GPUs; only world_size 1 is "
                                  "available here (capi.permute_rows / scatter_rows are the local halves)")
    n_out = int(recv_offset[-1])
    x = inputs.reshape(-1, feat_dim).contiguous()
    if fwd_flag:
        if x.shape[0] != n_out:
            raise ValueError("with one GPU the received row count equals the sent row count")
        return capi.permute_rows(x, permutation)
    return capi.scatter_rows(x, permutation, num_out_rows=n_out)


def _needs_peers(name):
    def op(*args, **kwargs):
        raise NotImplementedError(f"npc.{name} talks to other GPUs over NCCL in the reference; "
                                  "this library builds one GPU's share only")
    op.__name__ = name
    return op


for _n in ("nccl_get_unique_id", "init", "alltoall", "crossmachine_load_subtensor", "srcdst_to_vir",
           "src_to_vir", "np_sample_and_shuffle", "sp_sample_and_shuffle", "sp_sample_shuffle_src",
           "mp_sample_shuffle", "sp_feat_shuffle", "mp_feat_shuffle_fwd", "mp_feat_shuffle_bwd"):
    globals()[_n] = _needs_peers(_n)
