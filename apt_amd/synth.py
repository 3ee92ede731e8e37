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


def rmat_csr_gpu(num_nodes, num_edges, seed, device="cuda:0", a=RMAT_A, b=RMAT_B, c=RMAT_C):
    """Large R-MAT graph built directly in CSR on the GPU, without a sort.

    R-MAT's recursive quadrant choice factorises over bits: row id u has
    probability prod_l (a+b if bit_l(u)==0 else c+d), and given the row the
    neighbour's bits are independent.  So row degrees are drawn as
    Poisson(E * p_u / Z) (ids >= num_nodes excluded, i.e. rejected) and every
    neighbour slot is then filled independently by apt_synth_rmat_fill.
    Neighbour lists are unsorted and may repeat an id (multigraph), which the
    samplers treat as distinct positions.

    -> (indptr int64[num_nodes+1], indices int64[E'], E' ~ num_edges)
    """
    import math

    import torch

    from . import capi

    d = 1.0 - a - b - c
    levels = max(1, int(math.ceil(math.log2(max(num_nodes, 2)))))
    gen = torch.Generator(device=device)
    gen.manual_seed(int(seed))
    l0, l1 = math.log(a + b), math.log(c + d)
    indptr = torch.zeros(num_nodes + 1, dtype=torch.int64, device=device)
    chunk = 1 << 24
    # normaliser over ids < num_nodes, in float64
    z = 0.0
    logp_chunks = []
    for s in range(0, num_nodes, chunk):
        u = torch.arange(s, min(s + chunk, num_nodes), dtype=torch.int64, device=device)
        pc = torch.zeros_like(u)
        for bit in range(levels):
            pc += (u >> bit) & 1
        logp = (levels - pc).to(torch.float64) * l0 + pc.to(torch.float64) * l1
        z += float(torch.exp(logp).sum().item())
        logp_chunks.append((s, logp.to(torch.float32)))
        del u, pc, logp
    scale = math.log(num_edges) - math.log(z)
    for s, logp in logp_chunks:
        rate = torch.exp(logp.to(torch.float64) + scale).to(torch.float32)
        deg = torch.poisson(rate, generator=gen).to(torch.int64)
        indptr[s + 1:s + 1 + deg.numel()] = deg
        del rate, deg
    del logp_chunks
    torch.cumsum(indptr, 0, out=indptr)
    total = int(indptr[-1].item())
    indices = torch.empty(total, dtype=torch.int64, device=device)
    thr0 = int(round(65536 * b / (a + b)))
    thr1 = int(round(65536 * d / (c + d)))
    capi.synth_rmat_fill(indptr, num_nodes, total, levels, seed, thr0, thr1, indices)
    return indptr, indices


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
