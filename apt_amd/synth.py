"""Synthetic inputs: R-MAT power-law graphs in CSR, feature tables, seeds.

The reference trains on ogbn-products / ogbn-papers100M partitions
(scripts/preprocess_dataset.py, npc_dataset/*/configs.json); those datasets are
not reachable here, so tests and the benchmark use seeded R-MAT graphs
(a=.57 b=.19 c=.19 d=.05) of the same shapes.

Row v of the CSR lists the sampled-from neighbours of v, exactly what the
reference gets from graph.adj_tensors("csc") (python/npc/utils/utils.py:311).
"""
import numpy as np

RMAT_A, RMAT_B, RMAT_C, RMAT_D = 0.57, 0.19, 0.19, 0.05


def rmat_edges_numpy(num_nodes, num_edges, seed, a=RMAT_A, b=RMAT_B, c=RMAT_C):
    """Classic recursive-quadrant R-MAT on the CPU (small graphs only).
    Endpoints >= num_nodes are redrawn; duplicate edges are removed.
    -> (row, col) int64 arrays."""
    rng = np.random.default_rng(seed)
    levels = max(1, int(np.ceil(np.log2(max(num_nodes, 2)))))
    row = np.empty(0, dtype=np.int64)
    col = np.empty(0, dtype=np.int64)
    want = num_edges
    for _ in range(64):
        m = int(want * 1.3) + 16
        r = np.zeros(m, dtype=np.int64)
        q = np.zeros(m, dtype=np.int64)
        for _l in range(levels):
            u = rng.random(m)
            rbit = (u >= a + b).astype(np.int64)
            cbit = (((u >= a) & (u < a + b)) | (u >= a + b + c)).astype(np.int64)
            r = (r << 1) | rbit
            q = (q << 1) | cbit
        ok = (r < num_nodes) & (q < num_nodes)
        row = np.concatenate([row, r[ok]])
        col = np.concatenate([col, q[ok]])
        key = np.unique(row * num_nodes + col)
        row, col = key // num_nodes, key % num_nodes
        if len(row) >= num_edges:
            break
        want = num_edges - len(row)
    if len(row) > num_edges:
        keep = np.sort(rng.choice(len(row), size=num_edges, replace=False))
        row, col = row[keep], col[keep]
    return row, col


def csr_from_edges(num_nodes, row, col):
    """-> (indptr int64[num_nodes+1], indices int64[E]); row-major, neighbour
    lists sorted by id."""
    order = np.lexsort((col, row))
    row, col = row[order], col[order]
    indptr = np.zeros(num_nodes + 1, dtype=np.int64)
    np.add.at(indptr, row + 1, 1)
    return np.cumsum(indptr), col.astype(np.int64)


def rmat_csr_numpy(num_nodes, num_edges, seed):
    row, col = rmat_edges_numpy(num_nodes, num_edges, seed)
    return csr_from_edges(num_nodes, row, col)


def _rmat_log_row_prob(lo, hi, levels, device, a, b, c):
    """log of the unnormalised R-MAT row probability of ids [lo, hi): every 0
    bit contributes a+b, every 1 bit c+d."""
    import math

    import torch

    d = 1.0 - a - b - c
    u = torch.arange(lo, hi, dtype=torch.int64, device=device)
    pc = torch.zeros_like(u)
    for bit in range(levels):
        pc += (u >> bit) & 1
    return (levels - pc).to(torch.float64) * math.log(a + b) + pc.to(torch.float64) * math.log(c + d)


def rmat_expected_degree(num_nodes, num_edges, device="cuda:0", a=RMAT_A, b=RMAT_B, c=RMAT_C,
                         lo=0, hi=None):
    """Expected row degree E * p_u / Z of ids [lo, hi) (float32 tensor)."""
    import math

    import torch

    levels = max(1, int(math.ceil(math.log2(max(num_nodes, 2)))))
    chunk = 1 << 24
    z = 0.0
    for s in range(0, num_nodes, chunk):
        z += float(torch.exp(_rmat_log_row_prob(s, min(s + chunk, num_nodes), levels, device, a, b, c)).sum())
    hi = num_nodes if hi is None else hi
    scale = math.log(num_edges) - math.log(z)
    out = torch.empty(hi - lo, dtype=torch.float32, device=device)
    for s in range(lo, hi, chunk):
        e = min(s + chunk, hi)
        out[s - lo:e - lo] = torch.exp(_rmat_log_row_prob(s, e, levels, device, a, b, c) + scale).to(torch.float32)
    return out


def rmat_csr_gpu(num_nodes, num_edges, seed, device="cuda:0", a=RMAT_A, b=RMAT_B, c=RMAT_C,
                 row_begin=0, num_rows=None):
    """Large R-MAT graph built directly in CSR on the GPU, without a sort.

    R-MAT's recursive quadrant choice factorises over bits: row id u has
    probability prod_l (a+b if bit_l(u)==0 else c+d), and given the row the
    neighbour's bits are independent.  So row degrees are drawn as
    Poisson(E * p_u / Z) (ids >= num_nodes excluded, i.e. rejected) and every
    neighbour slot is then filled independently by apt_synth_rmat_fill.
    Neighbour lists are unsorted and may repeat an id (multigraph), which the
    samplers treat as distinct positions.  row_begin / num_rows build only the
    rows of a contiguous-range partition (neighbour ids stay global).

    -> (indptr int64[rows+1], indices int64[E'], E' ~ num_edges * row mass)
    """
    import math

    import torch

    from . import capi

    d = 1.0 - a - b - c
    if num_rows is None:
        num_rows = num_nodes - row_begin
    levels = max(1, int(math.ceil(math.log2(max(num_nodes, 2)))))
    gen = torch.Generator(device=device)
    gen.manual_seed(int(seed) * 1000003 + int(row_begin))
    rate = rmat_expected_degree(num_nodes, num_edges, device, a, b, c, row_begin, row_begin + num_rows)
    indptr = torch.zeros(num_rows + 1, dtype=torch.int64, device=device)
    chunk = 1 << 24
    for s in range(0, num_rows, chunk):
        e = min(s + chunk, num_rows)
        indptr[s + 1:e + 1] = torch.poisson(rate[s:e], generator=gen).to(torch.int64)
    del rate
    torch.cumsum(indptr, 0, out=indptr)
    total = int(indptr[-1].item())
    indices = torch.empty(total, dtype=torch.int64, device=device)
    thr0 = int(round(65536 * b / (a + b)))
    thr1 = int(round(65536 * d / (c + d)))
    capi.synth_rmat_fill(indptr, row_begin, num_nodes, total, levels, seed, thr0, thr1, indices)
    return indptr, indices


def symmetrize_csr_numpy(indptr, indices):
    """Small graphs on the CPU: the simple, bidirected graph with a self-loop on every node that the
    reference trains on (scripts/load_data.py:13-17: remove_self_loop, add_self_loop, to_bidirected).
    -> (indptr, indices) with sorted rows."""
    n = len(indptr) - 1
    row = np.repeat(np.arange(n, dtype=np.int64), np.diff(indptr))
    col = np.asarray(indices, dtype=np.int64)
    loops = np.arange(n, dtype=np.int64)
    key = np.unique(np.concatenate([row * n + col, col * n + row, loops * n + loops]))
    return csr_from_edges(n, key // n, key % n)


def rmat_symmetric_csr_gpu(num_nodes, num_edges, seed, device="cuda:0", a=RMAT_A, b=RMAT_B, c=RMAT_C,
                           chunk_edges=1 << 27, stats=None):
    """Large R-MAT graph of the kind the reference trains on (scripts/load_data.py:13-17): simple,
    bidirected, a self-loop on every node, built on the GPU.

    num_edges // 2 forward edges are drawn as rmat_csr_gpu draws them; every edge is stored in both
    directions (in-degrees counted with one atomic per edge, reverse copies placed by tickets), every
    node gets a self-loop, then the rows are sorted and repeated entries merged, a range of rows at a
    time (keys (row << bits) | neighbour, torch.sort).  The result does not depend on scheduling.
    stats (dict, optional) receives forward_edges, entries_before_merge, merged_fraction.

    -> (indptr int64[num_nodes + 1], indices int64[E'], rows sorted by id, no repeats)
    """
    import math

    import torch

    from . import capi

    N = int(num_nodes)
    fwd_indptr, fwd_indices = rmat_csr_gpu(N, num_edges // 2, seed, device, a, b, c)
    in_deg = torch.zeros(N, dtype=torch.int64, device=device)
    capi.count_ids(fwd_indices, in_deg)
    indptr = torch.zeros(N + 1, dtype=torch.int64, device=device)
    torch.cumsum(fwd_indptr[1:] - fwd_indptr[:-1] + in_deg + 1, 0, out=indptr[1:])
    del in_deg
    total = int(indptr[-1].item())
    out = torch.empty(total, dtype=torch.int64, device=device)
    capi.synth_symmetrize_fill(fwd_indptr, fwd_indices, indptr, out)
    n_fwd = int(fwd_indices.numel())
    del fwd_indptr, fwd_indices
    # ranges of rows holding about chunk_edges entries each
    marks = torch.arange(0, total, int(chunk_edges), dtype=torch.int64, device=device)
    rows = torch.unique(torch.clamp(torch.searchsorted(indptr, marks, right=True) - 1, min=0))
    rows = torch.cat([rows, torch.tensor([N], dtype=torch.int64, device=device)])
    rows[0] = 0
    rows_h = rows.cpu().tolist()
    offs_h = indptr[rows].cpu().tolist()
    bits = max(1, int(math.ceil(math.log2(max(N, 2)))))
    mask = (1 << bits) - 1
    new_deg = torch.empty(N, dtype=torch.int64, device=device)
    w = 0
    for (r0, r1), (e0, e1) in zip(zip(rows_h[:-1], rows_h[1:]), zip(offs_h[:-1], offs_h[1:])):
        if r1 == r0:
            continue
        local = torch.repeat_interleave(torch.arange(r1 - r0, dtype=torch.int64, device=device),
                                        indptr[r0 + 1:r1 + 1] - indptr[r0:r1], output_size=e1 - e0)
        key = torch.sort((local << bits) | out[e0:e1]).values
        del local
        keep = torch.ones(e1 - e0, dtype=torch.bool, device=device)
        keep[1:] = key[1:] != key[:-1]
        key = key[keep]
        del keep
        new_deg[r0:r1] = torch.bincount(key >> bits, minlength=r1 - r0)
        out[w:w + key.numel()] = key & mask            # w <= e0: only entries already read are overwritten
        w += int(key.numel())
        del key
    torch.cumsum(new_deg, 0, out=indptr[1:])
    if stats is not None:
        stats.update(forward_edges=n_fwd, entries_before_merge=total, merged_fraction=1.0 - w / max(total, 1))
    return indptr, out[:w]


def random_features(num_rows, dim, dtype, seed, device="cuda:0"):
    """~N(0,1) feature table generated on the GPU in chunks."""
    import torch

    gen = torch.Generator(device=device)
    gen.manual_seed(int(seed))
    out = torch.empty((num_rows, dim), dtype=dtype, device=device)
    step = max(1, (1 << 28) // max(dim, 1))
    for s in range(0, num_rows, step):
        e = min(s + step, num_rows)
        out[s:e] = torch.randn((e - s, dim), generator=gen, device=device, dtype=torch.float32).to(dtype)
    return out


def partition_share(num_nodes, num_edges, parts, part, dim, dtype, cache_ratio, seed, device="cuda:0",
                    full_graph=None):
    """One GPU's share of a graph split into `parts` contiguous id ranges (the reference's partitioned
    layout: python/npc/utils/utils.py load_partition, src/cache_feats.cc:14-61, src/core.cc:102-125):
    the CSR rows of range `part` (neighbour ids stay global), the feature rows of that range, a cache
    of the `cache_ratio` hottest remote rows (largest expected degree; ties by id), the position map
    over all ids (-(i)-2 local row i, >= 0 cache row, -1 absent), the range bounds `min_vids` and the
    owner -> request-bucket map (bucket 0 = this GPU, the other owners 1.. in id order).
    full_graph: (indptr, indices) of the whole graph on the device; the share is then its rows [lo, hi)
    and the cache holds the remote rows of largest actual degree.  Without it the share's rows of the
    directed multigraph generator are drawn and the cache goes by expected degree.
    -> dict(lo, hi, indptr, indices, feats, cache, hot, pos_map, min_vids, remote_worker_map)"""
    import torch

    lo, hi = num_nodes * part // parts, num_nodes * (part + 1) // parts
    if full_graph is not None:
        g_indptr, g_indices = full_graph
        e0, e1 = int(g_indptr[lo].item()), int(g_indptr[hi].item())
        indptr = (g_indptr[lo:hi + 1] - e0).contiguous()
        indices = g_indices[e0:e1].clone()
        exp_deg = (g_indptr[1:] - g_indptr[:-1]).to(torch.float32)
    else:
        indptr, indices = rmat_csr_gpu(num_nodes, num_edges, seed, device, row_begin=lo, num_rows=hi - lo)
        exp_deg = rmat_expected_degree(num_nodes, num_edges, device)
    feats = random_features(hi - lo, dim, dtype, seed + 1, device)
    exp_deg[lo:hi] = -1.0
    n_cache = int((num_nodes - (hi - lo)) * cache_ratio)
    hot = torch.sort(exp_deg, descending=True, stable=True).indices[:n_cache].contiguous()
    del exp_deg
    cache = random_features(n_cache, dim, dtype, seed + 3, device)
    pos_map = torch.full((num_nodes,), -1, dtype=torch.int64, device=device)
    pos_map[lo:hi] = -torch.arange(hi - lo, dtype=torch.int64, device=device) - 2
    pos_map[hot] = torch.arange(n_cache, dtype=torch.int64, device=device)
    min_vids = torch.tensor([num_nodes * k // parts for k in range(parts + 1)], dtype=torch.int64, device=device)
    rwm, nxt = [0] * parts, 1
    for k in range(parts):
        if k != part:
            rwm[k] = nxt
            nxt += 1
    return dict(lo=lo, hi=hi, indptr=indptr, indices=indices, feats=feats, cache=cache, hot=hot, pos_map=pos_map,
                min_vids=min_vids, remote_worker_map=torch.tensor(rwm, dtype=torch.int64, device=device))
