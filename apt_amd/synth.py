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
