"""ctypes binding of libapt_hip.so (declared in include/apt_amd.h).

This is the only place Python touches the C ABI.  Arguments are torch tensors
used purely as device buffers: the functions pass data pointers, sizes and the
current HIP stream.  There is no CPU fallback: if the library is missing or a
tensor is not on the GPU the call raises.
"""
import ctypes as C
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libapt_hip.so")

_lib = None


class AptError(RuntimeError):
    """A C-ABI call returned a non-zero status."""


class CGraph(C.Structure):
    _fields_ = [("indptr", C.c_void_p), ("indices", C.c_void_p),
                ("row_begin", C.c_int64), ("num_rows", C.c_int64),
                ("cached_indptr", C.c_void_p), ("cached_indices", C.c_void_p),
                ("num_cached_rows", C.c_int64), ("adj_pos_map", C.c_void_p),
                ("num_total_nodes", C.c_int64)]


class CFeatStore(C.Structure):
    _fields_ = [("local_table", C.c_void_p), ("num_local_rows", C.c_int64),
                ("local_dim", C.c_int64), ("cache_table", C.c_void_p),
                ("num_cache_rows", C.c_int64), ("pos_map", C.c_void_p),
                ("num_total_nodes", C.c_int64), ("col_offset", C.c_int64),
                ("out_dim", C.c_int64), ("elem_size", C.c_int)]


MAX_HOPS, MAX_SLOTS = 8, 16


ABI_VERSION = 2          # APT_ABI_VERSION of include/apt_amd.h


class CBlockBuffers(C.Structure):    # apt_block_buffers
    _fields_ = [("coo_row", C.c_void_p), ("coo_col", C.c_void_p), ("csc_indptr", C.c_void_p),
                ("csr_indptr", C.c_void_p), ("csr_indices", C.c_void_p), ("csr_eids", C.c_void_p),
                ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t)]


class CBatchSlot(C.Structure):       # apt_batch_slot
    _fields_ = [("stream", C.c_void_p), ("nodes", C.c_void_p),
                ("neighbors", C.c_void_p * MAX_HOPS), ("relabeled", C.c_void_p * MAX_HOPS),
                ("counts", C.c_void_p * MAX_HOPS), ("sizes", C.c_void_p), ("rank_table", C.c_void_p),
                ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t), ("features", C.c_void_p),
                ("miss_count", C.c_void_p), ("request_sizes", C.c_void_p), ("request_offsets", C.c_void_p),
                ("request_ids", C.c_void_p), ("request_perm", C.c_void_p), ("request_workspace", C.c_void_p),
                ("request_workspace_bytes", C.c_size_t), ("blocks", CBlockBuffers * MAX_HOPS),
                ("block_edges", C.c_void_p)]


class CEpochDesc(C.Structure):       # apt_epoch_desc
    _fields_ = [("graph", CGraph), ("store", CFeatStore), ("batch", C.c_int64), ("num_hops", C.c_int),
                ("hop_fanouts", C.c_int * MAX_HOPS), ("replace", C.c_int), ("rank_table_len", C.c_int64),
                ("has_requests", C.c_int), ("request_pos_map", C.c_void_p), ("request_num_total_nodes", C.c_int64),
                ("remote_worker_map", C.c_void_p), ("min_vids", C.c_void_p), ("world_size", C.c_int),
                ("num_remote_workers", C.c_int), ("formats", C.c_int), ("num_slots", C.c_int),
                ("slots", CBatchSlot * MAX_SLOTS)]


class CEpochCost(C.Structure):       # apt_epoch_cost
    _fields_ = [("batches", C.c_int64), ("enqueue_seconds", C.c_double), ("wait_enqueue_seconds", C.c_double),
                ("wait_gpu_seconds", C.c_double), ("release_seconds", C.c_double)]


# every symbol include/apt_amd.h declares: name -> (restype, argtypes)
_P, _I64, _I, _U64, _SZ = C.c_void_p, C.c_int64, C.c_int, C.c_uint64, C.c_size_t
SYMBOLS = {
    "apt_last_error": (C.c_char_p, []),
    "apt_abi_version": (_I, []),
    "apt_set_tuning": (_I, [C.c_char_p, _I]),
    "apt_sample_neighbors": (_I, [C.POINTER(CGraph), _P, _I64, _P, _I, _I, _U64, _I, _P, _P, _P, _P]),
    "apt_relabel_workspace_bytes": (_SZ, [_I64]),
    "apt_relabel": (_I, [_P, _I64, _P, _P, _I64, _I64, _P, _P, _P, _P, _P, _SZ, _P]),
    "apt_relabel_ranked_max_items": (_I64, []),
    "apt_relabel_ranked_workspace_bytes": (_SZ, [_I64]),
    "apt_relabel_ranked": (_I, [_P, _I64, _P, _P, _I64, _I64, _I, _P, _I64, _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "apt_sample_neighbors_bidding": (_I, [C.POINTER(CGraph), _P, _I64, _P, _I, _I, _U64, _I, _P, _P, _P, _I, _P, _I64, _P,
                                          _P, _P, _SZ, _P]),
    "apt_relabel_static_max_items": (_I64, []),
    "apt_relabel_static": (_I, [_P, _I64, _P, _P, _I64, _I64, _P, _P, _P, _P]),
    "apt_gather_rows": (_I, [C.POINTER(CFeatStore), _P, _I64, _P, _P, _P, _P]),
    "apt_time_next_gather": (_I, [_P, _P]),
    "apt_permute_rows": (_I, [_P, _I64, _P, _I64, _I64, _I, _P, _P]),
    "apt_scatter_workspace_bytes": (C.c_size_t, [_I64]),
    "apt_scatter_rows": (_I, [_P, _P, _I64, _I64, _I, _P, _I64, _P, C.c_size_t, _P]),
    "apt_bucket_workspace_bytes": (_SZ, [_I64, _I]),
    "apt_cluster_permute": (_I, [_P, _I64, _P, _P, _I, _I64, _I, _I, _I, _P, _P, _P, _P, _P, _SZ, _P]),
    "apt_cluster_reqs": (_I, [_P, _I64, _P, _P, _I64, _P, _P, _I, _I, _P, _P, _P, _P, _P, _SZ, _P]),
    "apt_rank_table_bytes": (_SZ, [_I64]),
    "apt_rank_table_init": (_I, [_P, _SZ, _P]),
    "apt_minibatch_workspace_bytes": (_SZ, [_I64, C.POINTER(C.c_int), _I]),
    "apt_minibatch_workspace_init": (_I, [_P, _SZ, _P]),
    "apt_minibatch_capacity": (_I64, [_I64, C.POINTER(C.c_int), _I, _I]),
    "apt_minibatch_sample": (_I, [C.POINTER(CGraph), _P, _I64, C.POINTER(C.c_int), _I, _I, _U64, _P,
                                  _P, _I64, _P, C.POINTER(_P), C.POINTER(_P), C.POINTER(_P), _P, _P,
                                  _SZ, _P]),
    "apt_minibatch_sample_deferred": (_I, [C.POINTER(CGraph), _P, _I64, C.POINTER(C.c_int), _I, _I, _U64, _P,
                                           _P, _I64, _P, C.POINTER(_P), C.POINTER(_P), C.POINTER(_P), _P, _P,
                                           _SZ, _P, _P]),
    "apt_minibatch_lookup": (_I, [_P, _P]),
    "apt_gather_rows_with_lookup": (_I, [C.POINTER(CFeatStore), _P, _I64, _P, _P, _P, _P, _P]),
    "apt_count_ids": (_I, [_P, _I64, _P, _P, _I64, _P]),
    "apt_csr_row_degrees": (_I, [_P, _I64, _I64, _P, _I64, _P, _P]),
    "apt_csr_copy_rows": (_I, [_P, _P, _I64, _P, _I64, _P, _I64, _P, _P]),
    "apt_map_to_vir": (_I, [_P, _I64, _P, _I64, _I, _P, _I, _I64, _I, _I, _I, _P, _P]),
    "apt_vir_send_offset": (_I, [_I, _I64, _P, _I64, _P, _I64, _I, _P, _P]),
    "apt_block_workspace_bytes": (_SZ, [_I64, _I, _I64, _I]),
    "apt_block_formats": (_I, [_P, _I64, _P, _I, _I64, _P, _P, _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "apt_spmm_sum": (_I, [_I, _P, _P, _I64, _P, _I64, _P, _I64, _I, _P, _P, _P, _I, _P, _I64, _P, _P]),
    "apt_coo_is_grouped": (_I, [_P, _I64, _P, _P]),
    "apt_spmm_block": (_I, [_P, _I64, _P, _I, _P, _I64, _I64, _I, _I, _P, _P]),
    "apt_sddmm": (_I, [_I, _P, _P, _I64, _P, _I64, _P, _I64, _I64, _I, _P, _P, _P, _I, _P, _P]),
    "apt_gat_scores": (_I, [_P, _I64, _I, _I64, _I, _P, _P, _P]),
    "apt_gat_block": (_I, [_P, _I64, _P, _I, _P, _I64, _I, _I64, _I, _P, _P, C.c_float, _P, _P, _P]),
    "apt_gat_block_backward": (_I, [_P, _I64, _I, _P, _I64, _I, _I64, _I, _P, _P, C.c_float, _P, _P, _P, _P, _P, _P, _P]),
    "apt_spmm_heads": (_I, [_P, _P, _I64, _P, _I64, _P, _P, _I, _I64, _I, _I, _P, _I64, _P, _P, _P, _P]),
    "apt_time_next_sample": (_I, [_I, _P, _P]),
    "apt_epoch_create": (_I, [C.POINTER(CEpochDesc), C.POINTER(_P)]),
    "apt_epoch_begin": (_I, [_P, _P, _I64, _U64, _P]),
    "apt_epoch_next": (_I, [_P, C.POINTER(_I), _P, _P]),
    "apt_epoch_release": (_I, [_P, _P]),
    "apt_epoch_end": (_I, [_P]),
    "apt_epoch_destroy": (_I, [_P]),
    "apt_epoch_host_cost": (_I, [_P, C.POINTER(CEpochCost)]),
}

# every symbol include/apt_synth.h declares (libapt_bench.so: inputs and probes of the benchmark and the tests)
BENCH_LIB_PATH = os.path.join(_HERE, "libapt_bench.so")
BENCH_SYMBOLS = {
    "apt_synth_last_error": (C.c_char_p, []),
    "apt_synth_rmat_fill": (_I, [_P, _I64, _I64, _I64, _I64, _I, _U64, C.c_uint32, C.c_uint32, _P, _P]),
    "apt_synth_copy": (_I, [_P, _P, _I64, _P]),
    "apt_synth_random_access": (_I, [_I, _P, _I64, _I64, C.c_uint32, _P, _P]),
    "apt_synth_symmetrize_fill": (_I, [_P, _P, _I64, _I64, _P, _P, _P, _P]),
}
_bench_lib = None


def lib():
    """Load libapt_hip.so (built by apt_amd/build.py).  Raises if absent."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `python apt_amd/build.py` "
                "(hipcc, gfx950).  There is no CPU fallback.")
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        if L.apt_abi_version() != ABI_VERSION:
            raise ImportError(f"{LIB_PATH} has ABI version {L.apt_abi_version()}, these bindings are written against "
                              f"{ABI_VERSION}: rebuild it with `python apt_amd/build.py`")
        _lib = L
    return _lib


def check(status):
    if status != 0:
        raise AptError(f"[{status}] {lib().apt_last_error().decode()}")


def bench_lib():
    """Load libapt_bench.so (built by apt_amd/build.py beside libapt_hip.so).  Raises if absent."""
    global _bench_lib
    if _bench_lib is None:
        if not os.path.exists(BENCH_LIB_PATH):
            raise ImportError(f"{BENCH_LIB_PATH} is missing: build it with `python apt_amd/build.py`")
        L = C.CDLL(BENCH_LIB_PATH)
        for name, (res, args) in BENCH_SYMBOLS.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _bench_lib = L
    return _bench_lib


def bench_check(status):
    if status != 0:
        raise AptError(f"[{status}] {bench_lib().apt_synth_last_error().decode()}")


def set_tuning(key, value):
    check(lib().apt_set_tuning(key.encode(), int(value)))


def _ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream():
    """The current HIP stream of the current device as a pointer (the raw getter costs a fraction of
    building a torch.cuda.Stream object, which matters when a batch is a dozen calls)."""
    if _raw_stream is not None:
        return C.c_void_p(_raw_stream(torch.cuda.current_device()))
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _dev_i64(t, name):
    if t is None:
        return None
    if not (t.is_cuda and t.dtype == torch.int64 and t.is_contiguous()):
        raise TypeError(f"{name} must be a contiguous int64 tensor on the GPU "
                        f"(got {t.dtype}, {t.device}, contiguous={t.is_contiguous()})")
    return t


class Graph:
    """Device-resident CSR graph in the layout of apt_graph."""

    def __init__(self, indptr, indices, row_begin=0, cached_indptr=None, cached_indices=None,
                 adj_pos_map=None, num_total_nodes=None):
        self.indptr = _dev_i64(indptr, "indptr")
        self.indices = _dev_i64(indices, "indices")
        self.cached_indptr = _dev_i64(cached_indptr, "cached_indptr")
        self.cached_indices = _dev_i64(cached_indices, "cached_indices")
        self.adj_pos_map = _dev_i64(adj_pos_map, "adj_pos_map")
        self.row_begin = int(row_begin)
        self.num_rows = indptr.numel() - 1
        self.num_cached_rows = 0 if cached_indptr is None else cached_indptr.numel() - 1
        if num_total_nodes is None:
            num_total_nodes = (adj_pos_map.numel() if adj_pos_map is not None
                               else self.row_begin + self.num_rows)
        self.num_total_nodes = int(num_total_nodes)
        self.c = CGraph(_ptr(self.indptr), _ptr(self.indices), self.row_begin, self.num_rows,
                        _ptr(self.cached_indptr), _ptr(self.cached_indices),
                        self.num_cached_rows, _ptr(self.adj_pos_map), self.num_total_nodes)

    @property
    def device(self):
        return self.indptr.device


class FeatStore:
    """Device-resident feature tables in the layout of apt_feat_store."""

    def __init__(self, local_table, cache_table=None, pos_map=None, col_offset=0, out_dim=None,
                 num_total_nodes=None):
        if not (local_table.is_cuda and local_table.is_contiguous() and local_table.dim() == 2):
            raise TypeError("local_table must be a contiguous 2-D tensor on the GPU")
        if local_table.element_size() not in (2, 4):
            raise TypeError(f"unsupported feature dtype {local_table.dtype}")
        if cache_table is not None and cache_table.numel() == 0:
            cache_table = None
        if cache_table is not None:
            if not (cache_table.is_cuda and cache_table.is_contiguous()
                    and cache_table.dtype == local_table.dtype and cache_table.dim() == 2):
                raise TypeError("cache_table must be a contiguous 2-D GPU tensor of the local dtype")
            if pos_map is None:
                raise ValueError("a cache table needs a position map")
        self.local_table = local_table
        self.cache_table = cache_table
        self.pos_map = _dev_i64(pos_map, "pos_map")
        self.col_offset = int(col_offset)
        self.local_dim = local_table.shape[1]
        if out_dim is None:
            out_dim = cache_table.shape[1] if cache_table is not None else self.local_dim - self.col_offset
        self.out_dim = int(out_dim)
        if cache_table is not None and cache_table.shape[1] != self.out_dim:
            raise ValueError("cache_table width must equal out_dim")
        if num_total_nodes is None:
            num_total_nodes = pos_map.numel() if pos_map is not None else local_table.shape[0]
        self.num_total_nodes = int(num_total_nodes)
        self.dtype = local_table.dtype
        self.c = CFeatStore(_ptr(local_table), local_table.shape[0], self.local_dim,
                            _ptr(cache_table), 0 if cache_table is None else cache_table.shape[0],
                            _ptr(self.pos_map), self.num_total_nodes, self.col_offset,
                            self.out_dim, local_table.element_size())

    @property
    def device(self):
        return self.local_table.device


def sample_neighbors(graph, frontier, fanout, replace, rng_seed, hop, num_frontier_dev=None,
                     out_neighbors=None, out_counts=None, out_total=None, want_counts=True):
    """-> (neighbors int64[n*fanout] padded with -1, counts int64[n] or None)."""
    frontier = _dev_i64(frontier, "frontier")
    n = frontier.numel()
    if fanout <= 0:
        raise AptError(f"fanout {fanout} must be > 0")
    if out_neighbors is None:
        out_neighbors = torch.empty(n * fanout, dtype=torch.int64, device=frontier.device)
    if out_counts is None and want_counts:
        out_counts = torch.empty(n, dtype=torch.int64, device=frontier.device)
    check(lib().apt_sample_neighbors(C.byref(graph.c), _ptr(frontier), n, _ptr(num_frontier_dev),
                                     int(fanout), int(bool(replace)),
                                     int(rng_seed) & 0xFFFFFFFFFFFFFFFF, int(hop),
                                     _ptr(out_neighbors), _ptr(out_counts), _ptr(out_total),
                                     _stream()))
    return out_neighbors, out_counts


def relabel_workspace_bytes(num_items):
    return int(lib().apt_relabel_workspace_bytes(int(num_items)))


def relabel(seeds, neighbors, num_seeds_dev=None, neighbor_stride=0, unique=None, relabeled=None,
            num_unique_dev=None, workspace=None, sync=True):
    """-> (unique, relabeled, num_unique).  With sync=True `unique` is narrowed
    to the count and num_unique is an int; otherwise both buffers keep their
    capacity and num_unique is the device int64[1] tensor."""
    seeds = _dev_i64(seeds, "seeds")
    neighbors = _dev_i64(neighbors, "neighbors")
    dev = seeds.device
    ns, nn = seeds.numel(), neighbors.numel()
    if unique is None:
        unique = torch.empty(ns + nn, dtype=torch.int64, device=dev)
    if relabeled is None:
        relabeled = torch.empty(nn, dtype=torch.int64, device=dev)
    if num_unique_dev is None:
        num_unique_dev = torch.empty(1, dtype=torch.int64, device=dev)
    need = relabel_workspace_bytes(ns + nn)
    if need == 0:
        raise AptError(f"relabel: {ns + nn} items exceed the supported maximum")
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=dev)
    host = C.c_int64(-1)
    check(lib().apt_relabel(_ptr(seeds), ns, _ptr(num_seeds_dev), _ptr(neighbors), nn,
                            int(neighbor_stride), _ptr(unique), _ptr(relabeled),
                            _ptr(num_unique_dev), C.cast(C.pointer(host), C.c_void_p) if sync else None,
                            _ptr(workspace), workspace.numel(), _stream()))
    if sync:
        return unique[:host.value], relabeled, int(host.value)
    return unique, relabeled, num_unique_dev


class RankedRelabel:
    """apt_relabel_ranked with its rank table and workspace: relabel calls for ids below num_total_nodes.
    relabel(seeds, neighbors) -> (unique, relabeled, num_unique) like capi.relabel(sync=True); a call whose seeds
    are the tensor the previous call returned as `unique` continues that batch (the table still holds its ids)."""

    def __init__(self, num_total_nodes, device):
        self.table = rank_table(num_total_nodes, device)
        self.table_len = int(num_total_nodes)
        self.workspace = None
        self.counts = torch.zeros(2, dtype=torch.int64, device=device)
        # the unique list the last call returned (kept alive, so that its address cannot be given to another
        # tensor) and its (data_ptr, numel, version): seeds with the same identity continue that batch
        self._last, self._last_tensor = None, None
        torch.cuda.current_stream().synchronize()

    def _workspace_for(self, items, device):
        need = int(lib().apt_relabel_ranked_workspace_bytes(items))
        if need == 0:
            raise AptError(f"relabel_ranked: {items} items exceed the supported maximum")
        if self.workspace is None or self.workspace.numel() < need:
            self.workspace = torch.empty(max(need, 256) * 2, dtype=torch.uint8, device=device)
            check(lib().apt_minibatch_workspace_init(_ptr(self.workspace), self.workspace.numel(), _stream()))

    def sample_bidding(self, graph, frontier, fanout, replace, rng_seed, hop, continued, out_neighbors, slot_states,
                       num_frontier_dev=None, out_counts=None, out_total=None, num_outside_dev=None):
        """apt_sample_neighbors_bidding: one hop of sampling that places the bids of the relabel call that follows
        (enqueue(..., bids_placed=True) with slot_states as `relabeled`).  fanout <= 64."""
        frontier = _dev_i64(frontier, "frontier")
        n = frontier.numel()
        self._workspace_for(n + n * int(fanout), frontier.device)
        self._last = self._last_tensor = None
        check(lib().apt_sample_neighbors_bidding(C.byref(graph.c), _ptr(frontier), n, _ptr(num_frontier_dev), int(fanout),
                                                 int(bool(replace)), int(rng_seed) & 0xFFFFFFFFFFFFFFFF, int(hop),
                                                 _ptr(out_neighbors), _ptr(out_counts), _ptr(out_total),
                                                 int(bool(continued)), _ptr(self.table), self.table_len,
                                                 _ptr(slot_states), _ptr(num_outside_dev), _ptr(self.workspace),
                                                 self.workspace.numel(), _stream()))

    def enqueue(self, seeds, neighbors, continued, unique, relabeled, num_unique_dev, num_outside_dev,
                num_seeds_dev=None, neighbor_stride=0, bids_placed=False):
        """Asynchronous form with the caller's buffers and device-side sizes (as capi.relabel(sync=False)):
        num_unique_dev receives the count, num_outside_dev is incremented per id outside the table (device
        int64[1] each; the caller clears the second).  bids_placed: `neighbors` and `relabeled` come from
        sample_bidding on the same seeds."""
        seeds, neighbors = _dev_i64(seeds, "seeds"), _dev_i64(neighbors, "neighbors")
        self._workspace_for(seeds.numel() + neighbors.numel(), seeds.device)
        self._last = self._last_tensor = None
        check(lib().apt_relabel_ranked(_ptr(seeds), seeds.numel(), _ptr(num_seeds_dev), _ptr(neighbors),
                                       neighbors.numel(), int(neighbor_stride),
                                       int(bool(continued)) | (2 if bids_placed else 0), _ptr(self.table),
                                       self.table_len, _ptr(unique), _ptr(relabeled), _ptr(num_unique_dev),
                                       _ptr(num_outside_dev), None, _ptr(self.workspace), self.workspace.numel(),
                                       _stream()))

    def relabel(self, seeds, neighbors, continued=None):
        seeds, neighbors = _dev_i64(seeds, "seeds"), _dev_i64(neighbors, "neighbors")
        ns, nn = seeds.numel(), neighbors.numel()
        self._workspace_for(ns + nn, seeds.device)
        if continued is None:
            continued = self._last == (seeds.data_ptr(), ns, seeds._version)
        unique = torch.empty(ns + nn, dtype=torch.int64, device=seeds.device)
        relabeled = torch.empty(nn, dtype=torch.int64, device=seeds.device)
        host = (C.c_int64 * 2)(-1, -1)
        self._last = None
        self.counts.zero_()
        check(lib().apt_relabel_ranked(_ptr(seeds), ns, None, _ptr(neighbors), nn, 0, int(bool(continued)),
                                       _ptr(self.table), self.table_len, _ptr(unique), _ptr(relabeled),
                                       _ptr(self.counts[0:1]), _ptr(self.counts[1:2]), host,
                                       _ptr(self.workspace), self.workspace.numel(), _stream()))
        if host[1] != 0:
            raise AptError(f"relabel_ranked: {host[1]} ids are outside [0, {self.table_len})")
        unique = unique[:host[0]]
        self._last, self._last_tensor = (unique.data_ptr(), unique.numel(), unique._version), unique
        return unique, relabeled, int(host[0])


def gather_rows(store, index, num_index_dev=None, out=None, miss_count=None, pending=None):
    """out[r, :] = feature row of node index[r] -> out [n, out_dim].
    pending: what MinibatchPlan.launch(defer_lookup=True) left to do (a PendingLookup); it is carried out in the
    same launch."""
    index = _dev_i64(index, "index")
    n = index.numel()
    if out is None:
        out = torch.empty((n, store.out_dim), dtype=store.dtype, device=index.device)
    if pending is None:
        check(lib().apt_gather_rows(C.byref(store.c), _ptr(index), n, _ptr(num_index_dev), _ptr(out),
                                    _ptr(miss_count), _stream()))
    else:
        check(lib().apt_gather_rows_with_lookup(C.byref(store.c), _ptr(index), n, _ptr(num_index_dev), _ptr(out),
                                                _ptr(miss_count), C.addressof(pending.c), _stream()))
        pending.open = False
    return out


class PendingLookup:
    """Host-side description of a batch's last relabel pass (apt_pending_lookup)."""

    def __init__(self):
        self.c = (C.c_uint64 * 64)()
        self.open = False       # filled and not yet carried out

    def run(self):
        """Carries the pass out as a launch of its own (if it is still open)."""
        if self.open:
            check(lib().apt_minibatch_lookup(C.addressof(self.c), _stream()))
            self.open = False


def _rows2d(t, name):
    if not (t.is_cuda and t.is_contiguous() and t.dim() == 2 and t.element_size() in (2, 4)):
        raise TypeError(f"{name} must be a contiguous 2-D GPU tensor with 2- or 4-byte elements")
    return t


def permute_rows(table, perm, out=None):
    """out[i, :] = table[perm[i], :]"""
    table = _rows2d(table, "table")
    perm = _dev_i64(perm, "perm")
    n = perm.numel()
    if out is None:
        out = torch.empty((n, table.shape[1]), dtype=table.dtype, device=table.device)
    check(lib().apt_permute_rows(_ptr(table), table.shape[0], _ptr(perm), n, table.shape[1],
                                 table.element_size(), _ptr(out), _stream()))
    return out


def scatter_rows(table, perm, num_out_rows=None, out=None):
    """out[perm[i], :] = table[i, :]; rows nobody names are zero."""
    table = _rows2d(table, "table")
    perm = _dev_i64(perm, "perm")
    n = perm.numel()
    if n != table.shape[0]:
        raise AptError(f"scatter_rows: {table.shape[0]} rows but {n} destinations")
    if num_out_rows is None:
        num_out_rows = n
    ws = None
    if out is None:   # rows nobody names are flagged by the scatter and zeroed afterwards: no fill of the whole output
        out = torch.empty((num_out_rows, table.shape[1]), dtype=table.dtype, device=table.device)
        ws = torch.empty(int(lib().apt_scatter_workspace_bytes(int(num_out_rows))), dtype=torch.uint8,
                         device=table.device)
    check(lib().apt_scatter_rows(_ptr(table), _ptr(perm), n, table.shape[1], table.element_size(),
                                 _ptr(out), int(num_out_rows), _ptr(ws), ws.numel() if ws is not None else 0,
                                 _stream()))
    return out


def cluster_permute(ids, min_vids, num_buckets, id_offset=0, rank=0, node_beg=0, node_end=None,
                    n_dev=None):
    """-> (bucket_size, bucket_offset, sorted_ids, permutation), all on the GPU."""
    ids = _dev_i64(ids, "ids")
    min_vids = _dev_i64(min_vids, "min_vids")
    if min_vids.numel() < num_buckets + 1:
        raise AptError(f"min_vids has {min_vids.numel()} entries, {num_buckets + 1} needed")
    if node_end is None:
        node_end = num_buckets
    dev, n = ids.device, ids.numel()
    bs = torch.empty(num_buckets, dtype=torch.int64, device=dev)
    bo = torch.empty(num_buckets, dtype=torch.int64, device=dev)
    so = torch.empty(n, dtype=torch.int64, device=dev)
    pm = torch.empty(n, dtype=torch.int64, device=dev)
    need = int(lib().apt_bucket_workspace_bytes(n, int(num_buckets)))
    if need == 0:
        raise AptError(f"cluster_permute: unsupported size (n={n}, buckets={num_buckets})")
    ws = torch.empty(need, dtype=torch.uint8, device=dev)
    check(lib().apt_cluster_permute(_ptr(ids), n, _ptr(n_dev), _ptr(min_vids), int(num_buckets), int(id_offset),
                                    int(rank), int(node_beg), int(node_end), _ptr(bs), _ptr(bo),
                                    _ptr(so), _ptr(pm), _ptr(ws), ws.numel(), _stream()))
    return bs, bo, so, pm


def cluster_reqs(ids, feat_pos_map, remote_worker_map, min_vids, world_size, num_remote_workers,
                 n_dev=None, out=None, workspace=None):
    """-> (bucket_size, bucket_offset, sorted_ids, permutation), all on the GPU.
    `out` / `workspace` let a caller reuse buffers across batches."""
    ids = _dev_i64(ids, "ids")
    feat_pos_map = _dev_i64(feat_pos_map, "feat_pos_map")
    remote_worker_map = _dev_i64(remote_worker_map, "remote_worker_map")
    min_vids = _dev_i64(min_vids, "min_vids")
    if min_vids.numel() < world_size + 1 or remote_worker_map.numel() < world_size:
        raise AptError("cluster_reqs: min_vids / remote_worker_map shorter than world_size")
    dev, n = ids.device, ids.numel()
    if out is None:
        out = (torch.empty(num_remote_workers, dtype=torch.int64, device=dev),
               torch.empty(num_remote_workers, dtype=torch.int64, device=dev),
               torch.empty(n, dtype=torch.int64, device=dev),
               torch.empty(n, dtype=torch.int64, device=dev))
    bs, bo, so, pm = out
    need = int(lib().apt_bucket_workspace_bytes(n, int(num_remote_workers)))
    if need == 0:
        raise AptError(f"cluster_reqs: unsupported size (n={n}, buckets={num_remote_workers})")
    ws = workspace if workspace is not None else torch.empty(need, dtype=torch.uint8, device=dev)
    if ws.numel() < need:
        raise AptError("cluster_reqs: workspace too small")
    check(lib().apt_cluster_reqs(_ptr(ids), n, _ptr(n_dev), _ptr(feat_pos_map), feat_pos_map.numel(),
                                 _ptr(remote_worker_map), _ptr(min_vids), int(world_size),
                                 int(num_remote_workers), _ptr(bs), _ptr(bo), _ptr(so), _ptr(pm),
                                 _ptr(ws), ws.numel(), _stream()))
    return bs, bo, so, pm


def synth_rmat_fill(indptr, row_begin, num_nodes, num_edges, levels, seed, thr0, thr1, indices):
    indptr = _dev_i64(indptr, "indptr")
    indices = _dev_i64(indices, "indices")
    if indices.numel() < num_edges:
        raise AptError("synth_rmat_fill: buffer sizes do not match")
    bench_check(bench_lib().apt_synth_rmat_fill(_ptr(indptr), indptr.numel() - 1, int(row_begin), int(num_nodes),
                                                int(num_edges), int(levels),
                                                int(seed) & 0xFFFFFFFFFFFFFFFF, int(thr0), int(thr1),
                                                _ptr(indices), _stream()))
    return indices


def synth_symmetrize_fill(fwd_indptr, fwd_indices, indptr, out):
    """Rows of the symmetrised graph with a self-loop per node, unsorted (apt_synth_symmetrize_fill)."""
    fwd_indptr, fwd_indices = _dev_i64(fwd_indptr, "fwd_indptr"), _dev_i64(fwd_indices, "fwd_indices")
    indptr, out = _dev_i64(indptr, "indptr"), _dev_i64(out, "out")
    n = fwd_indptr.numel() - 1
    if indptr.numel() != n + 1:
        raise AptError("synth_symmetrize_fill: indptr must have as many entries as fwd_indptr")
    cursor = torch.zeros(n, dtype=torch.int32, device=out.device)
    bench_check(bench_lib().apt_synth_symmetrize_fill(_ptr(fwd_indptr), _ptr(fwd_indices), n, fwd_indices.numel(),
                                                      _ptr(indptr), _ptr(cursor), _ptr(out), _stream()))
    return out


def synth_random_access(mode, table, num_accesses, salt, sink):
    """One random 4-byte access per work item into `table` (apt_synth_random_access)."""
    bench_check(bench_lib().apt_synth_random_access(int(mode), _ptr(table), table.numel() * table.element_size(),
                                                    int(num_accesses), int(salt), _ptr(sink), _stream()))


def rank_table(num_total_nodes, device):
    """Allocates and initialises the node-indexed rank table of the fused
    mini-batch driver (uint32 per node, all 0xFFFFFFFF)."""
    nbytes = int(lib().apt_rank_table_bytes(int(num_total_nodes)))
    if nbytes == 0 and num_total_nodes != 0:
        raise AptError(f"rank table: {num_total_nodes} nodes not supported")
    t = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=device)
    check(lib().apt_rank_table_init(_ptr(t), t.numel(), _stream()))
    return t


class MinibatchPlan:
    """Argument block of apt_minibatch_sample for fixed (batch, hop_fanouts):
    capacities, buffers and the host-side pointer arrays."""

    def __init__(self, graph, batch, hop_fanouts, replace=False, want_counts=True, table=None):
        self.graph = graph
        self.batch = int(batch)
        self.fanouts = [int(f) for f in hop_fanouts]
        self.replace = bool(replace)
        H = len(self.fanouts)
        self._cf = (C.c_int * H)(*self.fanouts)
        dev = graph.device
        self.caps = [int(lib().apt_minibatch_capacity(self.batch, self._cf, H, h)) for h in range(H + 1)]
        if min(self.caps) < 0:
            raise AptError("minibatch plan: unsupported batch / fanouts")
        i64 = dict(dtype=torch.int64, device=dev)
        self.nodes = torch.empty(max(self.caps[H], 1), **i64)
        self.neighbors = [torch.empty(max(self.caps[h] * f, 1), **i64) for h, f in enumerate(self.fanouts)]
        self.relabeled = [torch.empty(max(self.caps[h] * f, 1), **i64) for h, f in enumerate(self.fanouts)]
        self.counts = [torch.empty(max(self.caps[h], 1), **i64) for h in range(H)] if want_counts else None
        self.sizes = torch.zeros(H + 2, **i64)
        self.pending = PendingLookup()
        self.rng_seed_dev = torch.zeros(1, **i64)
        self.table = table if table is not None else rank_table(graph.num_total_nodes, dev)
        self.table_len = graph.num_total_nodes
        need = int(lib().apt_minibatch_workspace_bytes(self.batch, self._cf, H))
        self.workspace = torch.empty(max(need, 256), dtype=torch.uint8, device=dev)
        check(lib().apt_minibatch_workspace_init(_ptr(self.workspace), self.workspace.numel(), _stream()))
        self._nb = (C.c_void_p * H)(*[t.data_ptr() for t in self.neighbors])
        self._rl = (C.c_void_p * H)(*[t.data_ptr() for t in self.relabeled])
        self._ct = (C.c_void_p * H)(*[t.data_ptr() for t in self.counts]) if want_counts else None
        # the table and workspace were initialised on the current stream; the plan may be used on any
        torch.cuda.current_stream().synchronize()

    def launch(self, seeds, rng_seed=None, defer_lookup=False):
        """Asynchronous.  rng_seed=None reads the seed from self.rng_seed_dev.
        defer_lookup: the relabel's last pass is left to the caller, who passes self.pending to gather_rows
        (or calls self.pending.run()); until then relabeled[] is not final."""
        seeds = _dev_i64(seeds, "seeds")
        if seeds.numel() != self.batch:
            raise AptError(f"expected {self.batch} seeds, got {seeds.numel()}")
        args = (C.byref(self.graph.c), _ptr(seeds), self.batch, self._cf, len(self.fanouts),
                int(self.replace), 0 if rng_seed is None else int(rng_seed) & 0xFFFFFFFFFFFFFFFF,
                _ptr(self.rng_seed_dev) if rng_seed is None else None, _ptr(self.table), self.table_len,
                _ptr(self.nodes), self._nb, self._rl, self._ct, _ptr(self.sizes), _ptr(self.workspace),
                self.workspace.numel(), _stream())
        self.pending.run()          # a pass still open from an earlier call goes first
        if defer_lookup:
            check(lib().apt_minibatch_sample_deferred(*args, C.addressof(self.pending.c)))
            self.pending.open = True
        else:
            check(lib().apt_minibatch_sample(*args))


class EpochDriver:
    """apt_epoch over the buffers of a list of MiniBatchPipeline objects (one slot each, fused driver) and
    their streams.  The pipelines keep owning the buffers; this object must not outlive them."""

    def __init__(self, pipes, streams):
        p0 = pipes[0]
        H = len(p0.fanouts)
        if len(pipes) > MAX_SLOTS or H > MAX_HOPS:
            raise AptError(f"epoch driver: at most {MAX_SLOTS} slots and {MAX_HOPS} hops")
        d = CEpochDesc()
        d.graph = p0.graph.c
        if p0.feat is not None:
            d.store = p0.feat.c
        d.batch, d.num_hops, d.replace = p0.plan.batch, H, int(p0.replace)
        for h, f in enumerate(p0.fanouts):
            d.hop_fanouts[h] = f
        d.rank_table_len = p0.plan.table_len
        rq = p0.requests
        if rq is not None:
            d.has_requests = 1
            d.request_pos_map = rq["feat_pos_map"].data_ptr()
            d.request_num_total_nodes = rq["feat_pos_map"].numel()
            d.remote_worker_map, d.min_vids = rq["remote_worker_map"].data_ptr(), rq["min_vids"].data_ptr()
            d.world_size, d.num_remote_workers = int(rq["world_size"]), int(rq["num_remote_workers"])
        d.formats = 1 if p0.formats is not None else 0
        d.num_slots = len(pipes)
        for k, (p, st) in enumerate(zip(pipes, streams)):
            s = d.slots[k]
            s.stream = st.cuda_stream
            s.nodes, s.sizes = p.plan.nodes.data_ptr(), p.plan.sizes.data_ptr()
            for h in range(H):
                s.neighbors[h], s.relabeled[h] = p.plan.neighbors[h].data_ptr(), p.plan.relabeled[h].data_ptr()
                s.counts[h] = p.plan.counts[h].data_ptr() if p.plan.counts is not None else None
            s.rank_table, s.workspace = p.plan.table.data_ptr(), p.plan.workspace.data_ptr()
            s.workspace_bytes = p.plan.workspace.numel()
            s.features = p.features.data_ptr() if p.features is not None else None
            s.miss_count = p.misses.data_ptr()
            if rq is not None:
                s.request_sizes, s.request_offsets = p.request_sizes.data_ptr(), p.request_offsets.data_ptr()
                s.request_ids, s.request_perm = p.request_ids.data_ptr(), p.request_perm.data_ptr()
                s.request_workspace, s.request_workspace_bytes = p.request_ws.data_ptr(), p.request_ws.numel()
            if p.formats is not None:
                s.block_edges = p.format_edges.data_ptr()
                for h, f in enumerate(p.formats):
                    b = s.blocks[h]
                    b.coo_row, b.coo_col, b.csc_indptr = f.coo_row.data_ptr(), f.coo_col.data_ptr(), f.csc_indptr.data_ptr()
                    if f.want_csr:
                        b.csr_indptr, b.csr_indices = f.csr_indptr.data_ptr(), f.csr_indices.data_ptr()
                        b.csr_eids = f.csr_eids.data_ptr()
                    b.workspace, b.workspace_bytes = f.workspace.data_ptr(), f.workspace.numel()
        self._desc, self._keep = d, (pipes, streams)
        self.num_hops = H
        self.formats = bool(d.formats)
        self.num_requests = d.num_remote_workers if rq is not None else 0
        self.handle = C.c_void_p()
        check(lib().apt_epoch_create(C.byref(d), C.byref(self.handle)))
        self._slot = C.c_int()
        self._sizes = (C.c_int64 * (2 * H + 2))()
        self._req = (C.c_int64 * max(self.num_requests, 1))()

    def begin(self, seeds, num_batches, rng_seed0, ready_event=None):
        seeds = _dev_i64(seeds, "seeds")
        if seeds.numel() < num_batches * self._desc.batch:
            raise AptError("epoch driver: fewer seeds than num_batches * batch")
        self._seeds = seeds                                  # stays alive for the epoch
        self._ready = ready_event
        check(lib().apt_epoch_begin(self.handle, _ptr(seeds), int(num_batches), int(rng_seed0) & 0xFFFFFFFFFFFFFFFF,
                                    C.c_void_p(ready_event.cuda_event) if ready_event is not None else None))

    def next(self):
        """Blocks until the next batch is complete -> (slot, sizes list, request sizes list or None, edge counts of
        the blocks' formats or None)."""
        check(lib().apt_epoch_next(self.handle, C.byref(self._slot), self._sizes,
                                   self._req if self.num_requests else None))
        H = self.num_hops
        sizes = list(self._sizes)
        return (self._slot.value, sizes[:H + 2], (list(self._req)[:self.num_requests] if self.num_requests else None),
                sizes[H + 2:] if self.formats else None)

    def release(self):
        check(lib().apt_epoch_release(self.handle, _stream()))

    def end(self):
        check(lib().apt_epoch_end(self.handle))

    def host_cost(self):
        """-> dict(batches, enqueue_seconds, wait_enqueue_seconds, wait_gpu_seconds) since the driver was created."""
        c = CEpochCost()
        check(lib().apt_epoch_host_cost(self.handle, C.byref(c)))
        return {k: getattr(c, k) for k, _ in CEpochCost._fields_}

    def close(self):
        if self.handle:
            lib().apt_epoch_destroy(self.handle)
            self.handle = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def synth_copy(src, dst):
    """dst := src with the plain copy kernel (counter calibration)."""
    nbytes = src.numel() * src.element_size()
    if dst.numel() * dst.element_size() != nbytes:
        raise AptError("synth_copy: size mismatch")
    bench_check(bench_lib().apt_synth_copy(_ptr(src), _ptr(dst), nbytes, _stream()))
    return dst


def _feat2d(t, name):
    if not (t.is_cuda and t.is_contiguous() and t.dim() == 2 and t.dtype in (torch.float32, torch.bfloat16)):
        raise TypeError(f"{name} must be a contiguous 2-D fp32 or bf16 GPU tensor")
    return t


def _segments(coo_offset, num_edges, device):
    if coo_offset is None:
        coo_offset = torch.tensor([0, num_edges], dtype=torch.int64, device=device)
    return _dev_i64(coo_offset, "coo_offset")


def spmm_sum(mode, row, col, x, num_out, edata=None, coo_offset=None, input_offset=None,
             output_offset=None, detect_grouped=True):
    """mode 0 copy_u, 1 copy_e, 2 u_mul_e -> fp32 [num_out, dim] (see apt_spmm_sum).
    detect_grouped: check on the device whether col is non-decreasing and, if so, skip the atomics for
    rows inside a wavefront's edges."""
    row, col, x = _dev_i64(row, "row"), _dev_i64(col, "col"), _feat2d(x, "input")
    if edata is not None:
        edata = _feat2d(edata, "edata")
        if edata.dtype != x.dtype or edata.shape != (row.numel(), x.shape[1]):
            raise AptError("spmm_sum: edata must be [E, dim] of the input dtype")
    if mode == 1 and x.shape[0] != row.numel():
        raise AptError("spmm_sum: copy_e needs one input row per edge")
    if row.numel() != col.numel():
        raise AptError("spmm_sum: row and col differ in length")
    coo = _segments(coo_offset, row.numel(), x.device)
    out = torch.zeros((num_out, x.shape[1]), dtype=torch.float32, device=x.device)
    grouped = None
    if detect_grouped:
        grouped = torch.empty(1, dtype=torch.int32, device=x.device)
        check(lib().apt_coo_is_grouped(_ptr(col), col.numel(), _ptr(grouped), _stream()))
    check(lib().apt_spmm_sum(int(mode), _ptr(row), _ptr(col), row.numel(), _ptr(x), x.shape[0], _ptr(edata),
                             x.shape[1], x.element_size(), _ptr(coo), _ptr(_dev_i64(input_offset, "input_offset")),
                             _ptr(_dev_i64(output_offset, "output_offset")), coo.numel() - 1, _ptr(out),
                             int(num_out), _ptr(grouped), _stream()))
    return out


def sddmm(op, row, col, lhs, rhs, coo_offset=None, lhs_offset=None, rhs_offset=None):
    """op 0 u_add_v, 1 u_mul_v -> fp32 [E, dim] (see apt_sddmm)."""
    row, col = _dev_i64(row, "row"), _dev_i64(col, "col")
    lhs, rhs = _feat2d(lhs, "lhs"), _feat2d(rhs, "rhs")
    if lhs.dtype != rhs.dtype or lhs.shape[1] != rhs.shape[1] or row.numel() != col.numel():
        raise AptError("sddmm: lhs/rhs dtype or width mismatch")
    coo = _segments(coo_offset, row.numel(), lhs.device)
    out = torch.empty((row.numel(), lhs.shape[1]), dtype=torch.float32, device=lhs.device)
    check(lib().apt_sddmm(int(op), _ptr(row), _ptr(col), row.numel(), _ptr(lhs), lhs.shape[0], _ptr(rhs),
                          rhs.shape[0], lhs.shape[1], lhs.element_size(), _ptr(coo),
                          _ptr(_dev_i64(lhs_offset, "lhs_offset")), _ptr(_dev_i64(rhs_offset, "rhs_offset")),
                          coo.numel() - 1, _ptr(out), _stream()))
    return out


def spmm_block(neighbors, num_dst, fanout, x, mean=False, num_dst_dev=None, out=None):
    """Sum (or mean) of x rows over a sampled block in its fixed-stride layout
    (see apt_spmm_block) -> fp32 [num_dst, dim]."""
    neighbors = _dev_i64(neighbors, "neighbors")
    x = _feat2d(x, "input")
    if neighbors.numel() < num_dst * fanout:
        raise AptError("spmm_block: neighbors shorter than num_dst * fanout")
    if out is None:
        out = torch.empty((num_dst, x.shape[1]), dtype=torch.float32, device=x.device)
    check(lib().apt_spmm_block(_ptr(neighbors), int(num_dst), _ptr(num_dst_dev), int(fanout), _ptr(x),
                               x.shape[0], x.shape[1], x.element_size(), int(bool(mean)), _ptr(out),
                               _stream()))
    return out


def count_ids(ids, freq, n_dev=None):
    """freq[ids] += 1 (in place), ids outside [0, len(freq)) ignored."""
    ids = _dev_i64(ids, "ids")
    freq = _dev_i64(freq, "freq")
    check(lib().apt_count_ids(_ptr(ids), ids.numel(), _ptr(n_dev), _ptr(freq), freq.numel(), _stream()))
    return freq


def csr_row_degrees(graph, rows):
    """Degree of every node of `rows` in the graph's main table (0 outside it)."""
    rows = _dev_i64(rows, "rows")
    deg = torch.empty(rows.numel(), dtype=torch.int64, device=rows.device)
    if rows.numel():
        check(lib().apt_csr_row_degrees(_ptr(graph.indptr), graph.row_begin, graph.num_rows, _ptr(rows),
                                        rows.numel(), _ptr(deg), _stream()))
    return deg


def csr_select_rows(graph, rows):
    """The adjacency rows of `rows` (node ids) as a CSR of their own ->
    (indptr int64[n+1], indices int64[sum of degrees]).  Reads the graph's main
    table only (not a cache registered on it)."""
    rows = _dev_i64(rows, "rows")
    n = rows.numel()
    dev = rows.device
    out_indptr = torch.zeros(n + 1, dtype=torch.int64, device=dev)
    torch.cumsum(csr_row_degrees(graph, rows), 0, out=out_indptr[1:])
    total = int(out_indptr[-1].item())
    out_indices = torch.empty(total, dtype=torch.int64, device=dev)
    check(lib().apt_csr_copy_rows(_ptr(graph.indptr), _ptr(graph.indices), graph.row_begin, _ptr(rows), n,
                                  _ptr(out_indptr), total, _ptr(out_indices), _stream()))
    return out_indptr, out_indices


class BlockFormats:
    """COO / CSC / CSR of one hop's fixed-stride block (apt_block_formats).
    Buffers are sized for the upper bounds and reused by every emit(); the edge
    count stays on the device (num_edges).  narrow() waits and cuts to size."""

    def __init__(self, num_dst, fanout, num_src, want_csr=True, device="cuda:0", num_edges=None):
        self.num_dst, self.fanout, self.num_src, self.want_csr = int(num_dst), int(fanout), int(num_src), want_csr
        i64 = dict(dtype=torch.int64, device=device)
        slots = max(self.num_dst * self.fanout, 1)
        self.coo_row, self.coo_col = torch.empty(slots, **i64), torch.empty(slots, **i64)
        self.csc_indptr = torch.empty(self.num_dst + 1, **i64)
        # the edge count stays on the device; a caller that reads several at once passes its own int64[1] view
        self.num_edges = torch.zeros(1, **i64) if num_edges is None else _dev_i64(num_edges, "num_edges")
        self.csr_indptr = torch.empty(self.num_src + 1, **i64) if want_csr else None
        self.csr_indices = torch.empty(slots, **i64) if want_csr else None
        self.csr_eids = torch.empty(slots, **i64) if want_csr else None
        need = int(lib().apt_block_workspace_bytes(self.num_dst, self.fanout, self.num_src, int(want_csr)))
        if need == 0 and slots > 1:
            raise AptError("block formats: sizes out of range")
        self.workspace = torch.empty(max(need, 256), dtype=torch.uint8, device=device)

    def emit(self, relabeled, num_dst_dev=None):
        """Asynchronous."""
        relabeled = _dev_i64(relabeled, "relabeled")
        if relabeled.numel() < self.num_dst * self.fanout:
            raise AptError("block formats: relabeled is shorter than num_dst * fanout")
        check(lib().apt_block_formats(_ptr(relabeled), self.num_dst, _ptr(num_dst_dev), self.fanout, self.num_src,
                                      _ptr(self.coo_row), _ptr(self.coo_col), _ptr(self.csc_indptr),
                                      _ptr(self.num_edges), _ptr(self.csr_indptr), _ptr(self.csr_indices),
                                      _ptr(self.csr_eids), _ptr(self.workspace), self.workspace.numel(), _stream()))
        return self

    def narrow(self, num_dst=None, num_src=None, num_edges=None):
        """-> dict of the formats cut to the real sizes (waits for the stream unless
        the edge count is given)."""
        e = int(self.num_edges.item()) if num_edges is None else int(num_edges)
        nd = self.num_dst if num_dst is None else int(num_dst)
        ns = self.num_src if num_src is None else int(num_src)
        out = dict(num_edges=e, coo_row=self.coo_row[:e], coo_col=self.coo_col[:e], csc_indptr=self.csc_indptr[:nd + 1])
        if self.want_csr:
            out.update(csr_indptr=self.csr_indptr[:ns + 1], csr_indices=self.csr_indices[:e], csr_eids=self.csr_eids[:e])
        return out


def block_formats(relabeled, num_dst, fanout, num_src, want_csr=True, num_dst_dev=None):
    """One-shot form of BlockFormats: allocates, emits, narrows."""
    f = BlockFormats(num_dst, fanout, num_src, want_csr, device=relabeled.device)
    nd = num_dst if num_dst_dev is None else int(num_dst_dev.item())
    return f.emit(relabeled, num_dst_dev).narrow(num_dst=nd)


def _f32(t, name):
    if t is None:
        return None
    if not (t.is_cuda and t.is_contiguous() and t.dtype == torch.float32):
        raise TypeError(f"{name} must be a contiguous fp32 GPU tensor")
    return t


def gat_scores(x, attn):
    """(x * attn).sum(-1): x [n, heads, dim] fp32 / bf16, attn [heads, dim] fp32 -> fp32 [n, heads]."""
    if not (x.is_cuda and x.is_contiguous() and x.dim() == 3 and x.dtype in (torch.float32, torch.bfloat16)):
        raise TypeError("x must be a contiguous [n, heads, dim] fp32 or bf16 GPU tensor")
    attn = _f32(attn, "attn")
    n, heads, dim = x.shape
    if tuple(attn.shape) != (heads, dim):
        raise AptError("gat_scores: attn must be [heads, dim]")
    out = torch.empty((n, heads), dtype=torch.float32, device=x.device)
    check(lib().apt_gat_scores(_ptr(x), n, heads, dim, x.element_size(), _ptr(attn), _ptr(out), _stream()))
    return out


def gat_block(neighbors, num_dst, fanout, ft, el, er, negative_slope=0.2, num_dst_dev=None, want_attn=False):
    """Edge-softmax aggregation of a GAT layer over a fixed-stride block (see
    apt_gat_block) -> fp32 [num_dst, heads, dim] (, attention [num_dst * fanout, heads])."""
    neighbors = _dev_i64(neighbors, "neighbors")
    if not (ft.is_cuda and ft.is_contiguous() and ft.dim() == 3 and ft.dtype in (torch.float32, torch.bfloat16)):
        raise TypeError("ft must be a contiguous [num_src, heads, dim] fp32 or bf16 GPU tensor")
    el, er = _f32(el, "el"), _f32(er, "er")
    num_src, heads, dim = ft.shape
    if neighbors.numel() < num_dst * fanout:
        raise AptError("gat_block: neighbors shorter than num_dst * fanout")
    if tuple(el.shape) != (num_src, heads) or tuple(er.shape) != (num_dst, heads):
        raise AptError("gat_block: el must be [num_src, heads] and er [num_dst, heads]")
    out = torch.empty((num_dst, heads, dim), dtype=torch.float32, device=ft.device)
    attn = torch.empty((num_dst * fanout, heads), dtype=torch.float32, device=ft.device) if want_attn else None
    check(lib().apt_gat_block(_ptr(neighbors), int(num_dst), _ptr(num_dst_dev), int(fanout), _ptr(ft), num_src,
                              heads, dim, ft.element_size(), _ptr(el), _ptr(er), float(negative_slope), _ptr(out),
                              _ptr(attn), _stream()))
    return (out, attn) if want_attn else out


def map_to_vir(src, fanout, min_vids, world_size, rank=0, node_beg=0, node_end=None, id_offset=0, dst=None,
               num_dst=None):
    """Virtual-node ids of SP mode (see apt_map_to_vir).  dst given: [dst part, src part]
    as srcdst_to_vir; else num_dst must be given, as src_to_vir."""
    src = _dev_i64(src, "src")
    dst = _dev_i64(dst, "dst")
    min_vids = _dev_i64(min_vids, "min_vids")
    if min_vids.numel() < world_size + 1:
        raise AptError("map_to_vir: min_vids needs world_size + 1 entries")
    nd = dst.numel() if dst is not None else int(num_dst)
    out = torch.empty((nd if dst is not None else 0) + src.numel(), dtype=torch.int64, device=src.device)
    check(lib().apt_map_to_vir(_ptr(dst), nd, _ptr(src), src.numel(), int(fanout), _ptr(min_vids), int(world_size),
                               int(id_offset), int(rank), int(node_beg),
                               int(world_size if node_end is None else node_end), _ptr(out), _stream()))
    return out


def vir_send_offset(world_size, base, sorted_nodes, unique_nodes, with_dst=False):
    sorted_nodes, unique_nodes = _dev_i64(sorted_nodes, "sorted_nodes"), _dev_i64(unique_nodes, "unique_nodes")
    out = torch.empty(world_size * (3 if with_dst else 2) + 1, dtype=torch.int64, device=sorted_nodes.device)
    check(lib().apt_vir_send_offset(int(world_size), int(base), _ptr(sorted_nodes), sorted_nodes.numel(),
                                    _ptr(unique_nodes), unique_nodes.numel(), int(with_dst), _ptr(out), _stream()))
    return out


def gat_block_backward(neighbors, num_dst, fanout, ft, el, er, negative_slope, attn, d_out, csc_indptr, num_edges):
    """Edge half of the backward pass of gat_block -> (a_edge [E, heads], dz_edge [E, heads], d_er [num_dst, heads])."""
    num_src, heads, dim = ft.shape
    dev = ft.device
    a_edge = torch.empty((num_edges, heads), dtype=torch.float32, device=dev)
    dz_edge = torch.empty((num_edges, heads), dtype=torch.float32, device=dev)
    d_er = torch.empty((num_dst, heads), dtype=torch.float32, device=dev)
    check(lib().apt_gat_block_backward(_ptr(_dev_i64(neighbors, "neighbors")), int(num_dst), int(fanout), _ptr(ft),
                                       num_src, heads, dim, ft.element_size(), _ptr(_f32(el, "el")),
                                       _ptr(_f32(er, "er")), float(negative_slope), _ptr(_f32(attn, "attn")),
                                       _ptr(_f32(d_out, "d_out")), _ptr(_dev_i64(csc_indptr, "csc_indptr")),
                                       _ptr(a_edge), _ptr(dz_edge), _ptr(d_er), _stream()))
    return a_edge, dz_edge, d_er


def spmm_heads(row, col, x, head_weights, num_out, weight_row=None, grouped=False, head_weights2=None,
               out_indptr=None, out=None, out2=None):
    """out[col[e], h, :] += head_weights[w(e), h] * x[row[e], h, :], w(e) = weight_row[e] or e;
    x [n, heads, head_dim] (or [n, dim]: one head) -> fp32 of the same trailing shape with num_out rows.
    head_weights None = all ones.  grouped: edges with equal col are consecutive.  head_weights2: also
    returns out2[col[e], h] += head_weights2[w(e), h].  out_indptr (with grouped): CSR offsets of col; the
    outputs are then not zero-filled first (the library zeroes the rows it has to)."""
    row, col = _dev_i64(row, "row"), _dev_i64(col, "col")
    weight_row, out_indptr = _dev_i64(weight_row, "weight_row"), _dev_i64(out_indptr, "out_indptr")
    if x.dim() == 2:
        x = x.unsqueeze(1)
        flat = True
    else:
        flat = False
    n, heads, hd = x.shape
    w = _f32(head_weights, "head_weights")
    if not x.is_contiguous() or x.dtype not in (torch.float32, torch.bfloat16):
        raise AptError("spmm_heads: x must be a contiguous fp32 or bf16 tensor")
    if w is not None:
        if w.dim() != 2 or w.shape[1] != heads:
            raise AptError("spmm_heads: head_weights must be [*, heads]")
        if weight_row is None and w.shape[0] != row.numel():
            raise AptError("spmm_heads: head_weights needs one row per edge")
    if out_indptr is not None and (not grouped or out_indptr.numel() != num_out + 1):
        raise AptError("spmm_heads: out_indptr needs grouped edges and num_out + 1 entries")
    make = torch.empty if out_indptr is not None else torch.zeros
    if out is None:
        out = make((num_out, heads, hd), dtype=torch.float32, device=x.device)
    elif out.numel() != num_out * heads * hd or out.dtype != torch.float32 or not out.is_contiguous():
        raise AptError("spmm_heads: out must be a contiguous fp32 tensor of num_out rows")
    else:
        out = out.view(num_out, heads, hd)
    if head_weights2 is not None:
        head_weights2 = _f32(head_weights2, "head_weights2")
        if head_weights2.dim() != 2 or head_weights2.shape[1] != heads:
            raise AptError("spmm_heads: head_weights2 must be [*, heads]")
        if out2 is None:
            out2 = make((num_out, heads), dtype=torch.float32, device=x.device)
    check(lib().apt_spmm_heads(_ptr(row), _ptr(col), row.numel(), _ptr(x), n, _ptr(w), _ptr(weight_row), heads,
                               heads * hd, x.element_size(), int(grouped), _ptr(out), num_out, _ptr(head_weights2),
                               _ptr(out2), _ptr(out_indptr), _stream()))
    if flat:
        out = out.squeeze(1)
    return out if out2 is None else (out, out2)
