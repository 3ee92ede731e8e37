"""ctypes front end of oracle/liborc.so (built from oracle/oracle.c).

TEST INFRASTRUCTURE ONLY: the checker for the HIP library and the CPU baseline
that bench.py reports.  All arrays are numpy, C-contiguous; ids are int64.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liborc.so")

__all__ = [
    "build", "lib", "philox4x32_10", "draw64", "bounded", "Graph", "FeatStore",
    "sample_neighbors", "sample_positions", "relabel", "gather_rows",
    "permute_rows", "scatter_rows", "cluster_permute", "cluster_reqs",
    "set_threads", "max_threads", "sample_blocks", "spmm_sum", "spmm_csr", "sddmm", "count_ids", "csr_select_rows", "block_formats", "gat_scores", "gat_block", "map_to_vir", "vir_send_offset",
]


def build(force=False):
    """Compile oracle.c with gcc (a few seconds)."""
    src = os.path.join(_HERE, "oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liborc.so"],
                              stdout=subprocess.DEVNULL)
    return _SO


_lib = None


class _CGraph(C.Structure):
    _fields_ = [("indptr", C.c_void_p), ("indices", C.c_void_p),
                ("row_begin", C.c_int64), ("num_rows", C.c_int64),
                ("cached_indptr", C.c_void_p), ("cached_indices", C.c_void_p),
                ("num_cached_rows", C.c_int64), ("adj_pos_map", C.c_void_p),
                ("num_total_nodes", C.c_int64)]


class _CFeat(C.Structure):
    _fields_ = [("local_table", C.c_void_p), ("num_local_rows", C.c_int64),
                ("local_dim", C.c_int64), ("cache_table", C.c_void_p),
                ("num_cache_rows", C.c_int64), ("pos_map", C.c_void_p),
                ("num_total_nodes", C.c_int64), ("col_offset", C.c_int64),
                ("out_dim", C.c_int64), ("elem_size", C.c_int)]


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = C.CDLL(_SO)
        L.orc_draw64.restype = C.c_uint64
        L.orc_draw64.argtypes = [C.c_uint64, C.c_int64, C.c_int, C.c_uint32]
        L.orc_bounded.restype = C.c_uint64
        L.orc_bounded.argtypes = [C.c_uint64, C.c_uint64]
        L.orc_sample_neighbors.restype = C.c_int64
        L.orc_sample_positions.restype = C.c_int64
        L.orc_sample_positions.argtypes = [C.c_int64, C.c_int, C.c_int, C.c_uint64,
                                           C.c_int64, C.c_int, C.c_void_p]
        L.orc_relabel.restype = C.c_int64
        L.orc_gather_rows.restype = C.c_int64
        L.orc_set_threads.argtypes = [C.c_int]
        _lib = L
    return _lib


def set_threads(t):
    lib().orc_set_threads(int(t))


def max_threads():
    return int(lib().orc_max_threads())


def _i64(a):
    a = np.ascontiguousarray(a, dtype=np.int64)
    return a


def _p(a):
    return None if a is None else C.c_void_p(a.ctypes.data)


def philox4x32_10(ctr, key):
    c = np.asarray(ctr, dtype=np.uint32).copy()
    k = np.asarray(key, dtype=np.uint32).copy()
    o = np.zeros(4, dtype=np.uint32)
    lib().orc_philox4x32_10(_p(c), _p(k), _p(o))
    return o


def draw64(rng_seed, node, hop, slot):
    return int(lib().orc_draw64(rng_seed, node, hop, slot))


def bounded(r, n):
    return int(lib().orc_bounded(r, n))


class Graph:
    """Host copy of a graph in the layout of apt_graph (include/apt_amd.h)."""

    def __init__(self, indptr, indices, row_begin=0, cached_indptr=None,
                 cached_indices=None, adj_pos_map=None, num_total_nodes=None):
        self.indptr = _i64(indptr)
        self.indices = _i64(indices)
        self.row_begin = int(row_begin)
        self.num_rows = len(self.indptr) - 1
        self.cached_indptr = None if cached_indptr is None else _i64(cached_indptr)
        self.cached_indices = None if cached_indices is None else _i64(cached_indices)
        self.num_cached_rows = 0 if cached_indptr is None else len(self.cached_indptr) - 1
        self.adj_pos_map = None if adj_pos_map is None else _i64(adj_pos_map)
        if num_total_nodes is None:
            num_total_nodes = (len(self.adj_pos_map) if adj_pos_map is not None
                               else self.row_begin + self.num_rows)
        self.num_total_nodes = int(num_total_nodes)

    def c(self):
        return _CGraph(_p(self.indptr), _p(self.indices), self.row_begin, self.num_rows,
                       _p(self.cached_indptr), _p(self.cached_indices),
                       self.num_cached_rows, _p(self.adj_pos_map), self.num_total_nodes)


class FeatStore:
    """Host copy of feature tables in the layout of apt_feat_store."""

    def __init__(self, local_table, cache_table=None, pos_map=None, col_offset=0,
                 out_dim=None, num_total_nodes=None):
        self.local_table = np.ascontiguousarray(local_table)
        self.cache_table = None if cache_table is None else np.ascontiguousarray(cache_table)
        self.pos_map = None if pos_map is None else _i64(pos_map)
        self.col_offset = int(col_offset)
        self.local_dim = self.local_table.shape[1]
        if out_dim is None:
            out_dim = (self.cache_table.shape[1] if self.cache_table is not None
                       and self.cache_table.shape[0] > 0 else self.local_dim - self.col_offset)
        self.out_dim = int(out_dim)
        self.elem_size = self.local_table.dtype.itemsize
        if num_total_nodes is None:
            num_total_nodes = len(self.pos_map) if self.pos_map is not None else self.local_table.shape[0]
        self.num_total_nodes = int(num_total_nodes)

    def c(self):
        ct = self.cache_table
        return _CFeat(_p(self.local_table), self.local_table.shape[0], self.local_dim,
                      _p(ct), 0 if ct is None else ct.shape[0], _p(self.pos_map),
                      self.num_total_nodes, self.col_offset, self.out_dim, self.elem_size)


def sample_neighbors(graph, frontier, fanout, replace, rng_seed, hop):
    """-> (neighbors int64[n*fanout] padded with -1, counts int64[n])."""
    f = _i64(frontier)
    out = np.empty(len(f) * fanout, dtype=np.int64)
    cnt = np.empty(len(f), dtype=np.int64)
    g = graph.c()
    lib().orc_sample_neighbors(C.byref(g), _p(f), C.c_int64(len(f)), C.c_int(fanout),
                               C.c_int(int(bool(replace))), C.c_uint64(rng_seed),
                               C.c_int(hop), _p(out), _p(cnt))
    return out, cnt


def sample_positions(deg, fanout, replace, rng_seed, node, hop):
    out = np.empty(fanout, dtype=np.int64)
    c = lib().orc_sample_positions(deg, fanout, int(bool(replace)), rng_seed, node, hop, _p(out))
    return out[:c]


def relabel(seeds, neighbors):
    """-> (unique int64[U], relabeled int64[len(neighbors)])."""
    s = _i64(seeds)
    nb = _i64(neighbors)
    uniq = np.empty(len(s) + len(nb), dtype=np.int64)
    rel = np.empty(len(nb), dtype=np.int64)
    u = lib().orc_relabel(_p(s), C.c_int64(len(s)), _p(nb), C.c_int64(len(nb)), _p(uniq), _p(rel))
    return uniq[:u].copy(), rel


def gather_rows(store, index):
    """-> (out [n, out_dim], number of requests that were not present)."""
    idx = _i64(index)
    out = np.empty((len(idx), store.out_dim), dtype=store.local_table.dtype)
    st = store.c()
    miss = lib().orc_gather_rows(C.byref(st), _p(idx), C.c_int64(len(idx)), _p(out))
    return out, int(miss)


def permute_rows(table, perm):
    t = np.ascontiguousarray(table)
    p = _i64(perm)
    out = np.empty((len(p), t.shape[1]), dtype=t.dtype)
    lib().orc_permute_rows(_p(t), _p(p), C.c_int64(len(p)), C.c_int64(t.shape[1]),
                           C.c_int(t.dtype.itemsize), _p(out))
    return out


def scatter_rows(table, perm, num_out_rows=None):
    t = np.ascontiguousarray(table)
    p = _i64(perm)
    out = np.zeros((num_out_rows or len(p), t.shape[1]), dtype=t.dtype)
    lib().orc_scatter_rows(_p(t), _p(p), C.c_int64(len(p)), C.c_int64(t.shape[1]),
                           C.c_int(t.dtype.itemsize), _p(out))
    return out


def cluster_permute(ids, min_vids, num_buckets, id_offset=0, rank=0, node_beg=0, node_end=None):
    """-> (bucket_size, bucket_offset, sorted_ids, permutation)."""
    v = _i64(ids)
    mv = _i64(min_vids)
    if node_end is None:
        node_end = num_buckets
    bs = np.zeros(num_buckets, dtype=np.int64)
    bo = np.zeros(num_buckets, dtype=np.int64)
    so = np.empty(len(v), dtype=np.int64)
    pm = np.empty(len(v), dtype=np.int64)
    lib().orc_cluster_permute(_p(v), C.c_int64(len(v)), _p(mv), C.c_int(num_buckets),
                              C.c_int64(id_offset), C.c_int(rank), C.c_int(node_beg),
                              C.c_int(node_end), _p(bs), _p(bo), _p(so), _p(pm))
    return bs, bo, so, pm


def cluster_reqs(ids, feat_pos_map, remote_worker_map, min_vids, world_size, num_remote_workers):
    """-> (bucket_size, bucket_offset, sorted_ids, permutation)."""
    v = _i64(ids)
    fm = _i64(feat_pos_map)
    rw = _i64(remote_worker_map)
    mv = _i64(min_vids)
    bs = np.zeros(num_remote_workers, dtype=np.int64)
    bo = np.zeros(num_remote_workers, dtype=np.int64)
    so = np.empty(len(v), dtype=np.int64)
    pm = np.empty(len(v), dtype=np.int64)
    lib().orc_cluster_reqs(_p(v), C.c_int64(len(v)), _p(fm), C.c_int64(len(fm)), _p(rw), _p(mv),
                           C.c_int(world_size), C.c_int(num_remote_workers), _p(bs), _p(bo),
                           _p(so), _p(pm))
    return bs, bo, so, pm


def sample_blocks(graph, seeds, hop_fanouts, replace, rng_seed):
    """Multi-hop driver restating python/npc/sampler.py:187-203,358-364 (DP
    branch): hop h samples the current frontier with hop_fanouts[h] (the
    caller has already reversed the reference's k-hop..1-hop list), relabels,
    and the unique ids become the next frontier.

    -> (input_nodes, blocks) with blocks outermost-first; each block is a dict
    with seeds, neighbors (padded), counts, unique, relabeled (padded).
    """
    frontier = _i64(seeds)
    blocks = []
    for h, f in enumerate(hop_fanouts):
        nbr, cnt = sample_neighbors(graph, frontier, f, replace, rng_seed, h)
        uniq, rel = relabel(frontier, nbr)
        blocks.insert(0, dict(seeds=frontier, neighbors=nbr, counts=cnt, unique=uniq,
                              relabeled=rel, fanout=f))
        frontier = uniq
    return frontier, blocks


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def spmm_sum(mode, row, col, x, num_out, edata=None, coo_offset=None, input_offset=None,
             output_offset=None):
    """mode 0 copy_u, 1 copy_e, 2 u_mul_e -> float32 [num_out, dim]."""
    row, col, x = _i64(row), _i64(col), _f32(x)
    E, dim = len(row), x.shape[1]
    coo = _i64([0, E] if coo_offset is None else coo_offset)
    nseg = len(coo) - 1
    io = None if input_offset is None else _i64(input_offset)
    oo = None if output_offset is None else _i64(output_offset)
    ed = None if edata is None else _f32(edata)
    out = np.zeros((num_out, dim), dtype=np.float32)
    lib().orc_spmm_sum(C.c_int(mode), _p(row), _p(col), C.c_int64(E), _p(x), _p(ed), C.c_int64(dim),
                       _p(coo), _p(io), _p(oo), C.c_int(nseg), _p(out), C.c_int64(num_out))
    return out


def spmm_csr(indptr, indices, x, eids=None, col_scale=None, head_weights=None, head_weights2=None, heads=1):
    """out[r] = sum over CSR row r's edges of col_scale[idx] * head_weights[w(e), h] * x[idx]
    -> float32 [rows, dim] (and [rows, heads] with head_weights2); x is [n, dim], dim = heads * head_dim."""
    indptr, indices, x = _i64(indptr), _i64(indices), _f32(x)
    rows, dim = len(indptr) - 1, x.shape[1]
    ei = None if eids is None else _i64(eids)
    cs = None if col_scale is None else _f32(col_scale)
    w = None if head_weights is None else _f32(head_weights)
    w2 = None if head_weights2 is None else _f32(head_weights2)
    out = np.zeros((rows, dim), dtype=np.float32)
    out2 = None if w2 is None else np.zeros((rows, heads), dtype=np.float32)
    lib().orc_spmm_csr(_p(indptr), _p(indices), _p(ei), C.c_int64(rows), _p(x), C.c_int64(x.shape[0]),
                       C.c_int64(dim), _p(cs), _p(w), _p(w2), C.c_int(heads), _p(out), _p(out2))
    return out if out2 is None else (out, out2)


def sddmm(op, row, col, lhs, rhs, coo_offset=None, lhs_offset=None, rhs_offset=None):
    """op 0 u_add_v, 1 u_mul_v -> float32 [E, dim]."""
    row, col, lhs, rhs = _i64(row), _i64(col), _f32(lhs), _f32(rhs)
    E, dim = len(row), lhs.shape[1]
    coo = _i64([0, E] if coo_offset is None else coo_offset)
    lo = None if lhs_offset is None else _i64(lhs_offset)
    ro = None if rhs_offset is None else _i64(rhs_offset)
    out = np.zeros((E, dim), dtype=np.float32)
    lib().orc_sddmm(C.c_int(op), _p(row), _p(col), C.c_int64(E), _p(lhs), _p(rhs), C.c_int64(dim),
                    _p(coo), _p(lo), _p(ro), C.c_int(len(coo) - 1), _p(out))
    return out


def count_ids(ids, freq):
    """freq[ids] += 1 in place (ids outside the table ignored)."""
    v = _i64(ids)
    assert freq.dtype == np.int64 and freq.flags.c_contiguous
    lib().orc_count_ids(_p(v), C.c_int64(len(v)), _p(freq), C.c_int64(len(freq)))
    return freq


def csr_select_rows(graph, rows):
    """-> (indptr, indices) of the chosen nodes' adjacency rows."""
    r = _i64(rows)
    out_indptr = np.zeros(len(r) + 1, dtype=np.int64)
    lib().orc_csr_select_rows.restype = C.c_int64
    args = [_p(graph.indptr), _p(graph.indices), C.c_int64(graph.row_begin), C.c_int64(graph.num_rows),
            _p(r), C.c_int64(len(r)), _p(out_indptr)]
    total = lib().orc_csr_select_rows(*args, None)
    out_indices = np.empty(total, dtype=np.int64)
    lib().orc_csr_select_rows(*args, _p(out_indices))
    return out_indptr, out_indices


def block_formats(relabeled, num_dst, fanout, num_src, want_csr=True):
    """COO / CSC / CSR of a fixed-stride block -> dict of int64 arrays."""
    r = _i64(relabeled)
    assert len(r) == num_dst * fanout
    slots = max(len(r), 1)
    coo_row, coo_col = np.empty(slots, np.int64), np.empty(slots, np.int64)
    csc = np.empty(num_dst + 1, np.int64)
    csr = np.empty(num_src + 1, np.int64) if want_csr else None
    ci, ce = (np.empty(slots, np.int64), np.empty(slots, np.int64)) if want_csr else (None, None)
    lib().orc_block_formats.restype = C.c_int64
    e = lib().orc_block_formats(_p(r), C.c_int64(num_dst), C.c_int(fanout), C.c_int64(num_src), _p(coo_row),
                                _p(coo_col), _p(csc), _p(csr) if want_csr else None,
                                _p(ci) if want_csr else None, _p(ce) if want_csr else None)
    out = dict(num_edges=int(e), coo_row=coo_row[:e], coo_col=coo_col[:e], csc_indptr=csc)
    if want_csr:
        out.update(csr_indptr=csr, csr_indices=ci[:e], csr_eids=ce[:e])
    return out


def gat_scores(x, attn):
    """(x * attn).sum(-1): x [n, heads, dim], attn [heads, dim] -> float32 [n, heads]."""
    x, attn = _f32(x), _f32(attn)
    n, heads, dim = x.shape
    out = np.empty((n, heads), dtype=np.float32)
    lib().orc_gat_scores(_p(x), C.c_int64(n), C.c_int(heads), C.c_int64(dim), _p(attn), _p(out))
    return out


def gat_block(neighbors, num_dst, fanout, ft, el, er, negative_slope=0.2, want_attn=False):
    """GATConv aggregation over a fixed-stride block -> float32 [num_dst, heads, dim]
    (, attention [num_dst * fanout, heads])."""
    nbr, ft, el, er = _i64(neighbors), _f32(ft), _f32(el), _f32(er)
    num_src, heads, dim = ft.shape
    assert len(nbr) >= num_dst * fanout and el.shape == (num_src, heads) and er.shape == (num_dst, heads)
    out = np.empty((num_dst, heads, dim), dtype=np.float32)
    attn = np.empty((num_dst * fanout, heads), dtype=np.float32) if want_attn else None
    lib().orc_gat_block(_p(nbr), C.c_int64(num_dst), C.c_int(fanout), _p(ft), C.c_int64(num_src), C.c_int(heads),
                        C.c_int64(dim), _p(el), _p(er), C.c_double(negative_slope), _p(out), _p(attn))
    return (out, attn) if want_attn else out


def map_to_vir(src, fanout, min_vids, world_size, rank=0, node_beg=0, node_end=None, id_offset=0, dst=None,
               num_dst=None):
    src, mv = _i64(src), _i64(min_vids)
    d = None if dst is None else _i64(dst)
    nd = len(d) if d is not None else int(num_dst)
    out = np.empty((nd if d is not None else 0) + len(src), dtype=np.int64)
    lib().orc_map_to_vir(_p(d), C.c_int64(nd), _p(src), C.c_int64(len(src)), C.c_int(fanout), _p(mv),
                         C.c_int(world_size), C.c_int64(id_offset), C.c_int(rank), C.c_int(node_beg),
                         C.c_int(world_size if node_end is None else node_end), _p(out))
    return out


def vir_send_offset(world_size, base, sorted_nodes, unique_nodes, with_dst=False):
    s, u = _i64(sorted_nodes), _i64(unique_nodes)
    out = np.empty(world_size * (3 if with_dst else 2) + 1, dtype=np.int64)
    lib().orc_vir_send_offset(C.c_int(world_size), C.c_int64(base), _p(s), C.c_int64(len(s)), _p(u),
                              C.c_int64(len(u)), C.c_int(int(with_dst)), _p(out))
    return out
