"""Multi-hop mini-batch driver, the DP branch of MixedPSNeighborSampler
(reference python/npc/sampler.py:159-203,358-364) and create_dgl_block
(:76-91), without DGL: a block is a plain record of tensors."""
import torch

from . import ops


class Block:
    """Bipartite block of one hop.  Edge e goes from source row[e] (index into
    src_ids) to destination col[e] (index into the hop's seeds); the first
    num_dst source ids are the destination ids (reference sampler.py:76-91).
    relabeled / fanout: the same edges in the sampler's fixed-stride layout
    (relabeled[d * fanout + k], -1 = no edge), which the block aggregations read
    directly.  row / col (COO), csc() and csr(), DGL's three formats, are derived
    from it on first use: a forward pass over the fixed-stride layout never pays
    for them."""

    def __init__(self, num_src, num_dst, src_ids, relabeled, fanout, formats=None):
        self.num_src, self.num_dst = int(num_src), int(num_dst)
        self.src_ids = src_ids
        self.relabeled = relabeled
        self.fanout = int(fanout)
        self.formats = formats

    def __repr__(self):
        return f"Block(num_src={self.num_src}, num_dst={self.num_dst}, fanout={self.fanout})"

    def _formats(self, want_csr):
        if self.formats is None or (want_csr and "csr_indptr" not in self.formats):
            self.formats = ops.block_formats(self.relabeled, self.num_dst, self.fanout, self.num_src, want_csr)
        return self.formats

    @property
    def row(self):
        return self._formats(False)["coo_row"]

    @property
    def col(self):
        return self._formats(False)["coo_col"]

    def csc(self):
        """-> (indptr over destinations, source per edge, edge ids): the arguments
        of the reference's create_block_from_csc (sampler.py:44-56)."""
        f = self._formats(False)
        return f["csc_indptr"], f["coo_row"], torch.arange(f["num_edges"], device=self.relabeled.device)

    def csr(self):
        """-> (indptr over sources, destination per edge, edge ids)."""
        f = self._formats(True)
        return f["csr_indptr"], f["csr_indices"], f["csr_eids"]

    def number_of_src_nodes(self):
        return self.num_src

    def number_of_dst_nodes(self):
        return self.num_dst


def create_block(seeds, neighbors, fanout):
    """reference sampler.py:76-91 (create_dgl_block); -1 padded slots (rows
    with fewer than fanout neighbours) produce no edge."""
    unique, relabeled = ops.relabel_csc(seeds, neighbors)
    return _block(seeds.numel(), unique, relabeled, fanout)


def _block(num_dst, unique, relabeled, fanout, f=None):
    return Block(unique.numel(), num_dst, unique, relabeled, fanout, f)


class MixedPSNeighborSampler:
    """system="DP" only; fanouts are listed k-hop ... 1-hop as in the reference
    (python/npc/utils/utils.py:427-432) and walked in reverse, so the seeds are
    sampled with the last entry."""

    def __init__(self, rank, world_size, fanouts, system="DP", model=None, num_total_nodes=None,
                 shuffle_with_dst=False, debug_info=None, replace=True, rng_seed=None, fused=True, formats=False):
        if system != "DP":
            raise NotImplementedError(f"system {system!r} needs other GPUs; only 'DP' is available")
        self.rank, self.world_size = rank, world_size
        self.fanouts = list(fanouts)
        self.num_layers = len(self.fanouts)
        self.system = system
        self.replace = replace
        self.rng_seed = rng_seed
        self.fused = fused
        self.formats = bool(formats)      # fused: COO + CSC of every block inside the one call, else on first use
        self.batches = 0

    def sample(self, graph, seeds):
        """-> (input_nodes, output_nodes, blocks), blocks outermost first.  fused:
        one operator call for all hops; otherwise one sampling and one relabel
        call per hop as in the reference.  With an rng_seed both give the same
        batch."""
        output_nodes = seeds
        blocks = []
        if self.fused and (self.rng_seed is not None or not self.replace):
            seed = (self.rng_seed if self.rng_seed is not None else 0) + self.batches
            fan = list(reversed(self.fanouts))
            out = ops.sample_blocks(seeds, fan, self.replace, seed, formats=self.formats)
            sizes, nodes, hops = out[:3]
            for h, (_, relabeled, _) in enumerate(hops):
                blocks.insert(0, _block(sizes[h], nodes[:sizes[h + 1]], relabeled, fan[h],
                                        out[3][h] if self.formats else None))
            self.batches += 1
            return (nodes, output_nodes, blocks)
        for layer_id, fanout in enumerate(reversed(self.fanouts)):
            if self.replace and self.rng_seed is None:
                seeds, neighbors = ops.local_sample_one_layer(seeds, fanout)
            else:
                seed = (self.rng_seed if self.rng_seed is not None else 0) + self.batches
                neighbors, _ = ops.sample_neighbors(seeds, fanout, self.replace, seed, layer_id)
            block = create_block(seeds, neighbors, fanout)
            seeds = block.src_ids
            blocks.insert(0, block)
        self.batches += 1
        return (seeds, output_nodes, blocks)


def load_subtensor(args, sample_result):
    """reference python/npc/ops.py:528-600, DP branch: (blocks, input features)."""
    system = getattr(args, "system", "DP")
    if system != "DP":
        raise NotImplementedError(f"system {system!r} needs other GPUs; only 'DP' is available")
    return sample_result[2], ops.load_subtensor(sample_result[0])
