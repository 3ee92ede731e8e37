"""Multi-hop mini-batch driver, the DP branch of MixedPSNeighborSampler
(reference python/npc/sampler.py:159-203,358-364) and create_dgl_block
(:76-91), without DGL: a block is a plain record of COO tensors."""
from dataclasses import dataclass

import torch

from . import ops


@dataclass
class Block:
    """Bipartite block of one hop.  Edge e goes from source row[e] (index into
    src_ids) to destination col[e] (index into the hop's seeds); the first
    num_dst source ids are the destination ids (reference sampler.py:76-91)."""
    row: torch.Tensor
    col: torch.Tensor
    num_src: int
    num_dst: int
    src_ids: torch.Tensor

    def number_of_src_nodes(self):
        return self.num_src

    def number_of_dst_nodes(self):
        return self.num_dst


def create_block(seeds, neighbors, fanout):
    """reference sampler.py:76-91 (create_dgl_block); -1 padded slots (rows
    with fewer than fanout neighbours) produce no edge."""
    unique, relabeled = ops.relabel_csc(seeds, neighbors)
    col = torch.arange(seeds.numel(), device=relabeled.device).repeat_interleave(fanout)
    keep = relabeled >= 0
    if not bool(keep.all()):
        relabeled, col = relabeled[keep], col[keep]
    return Block(relabeled, col, unique.numel(), seeds.numel(), unique)


class MixedPSNeighborSampler:
    """system="DP" only; fanouts are listed k-hop ... 1-hop as in the reference
    (python/npc/utils/utils.py:427-432) and walked in reverse, so the seeds are
    sampled with the last entry."""

    def __init__(self, rank, world_size, fanouts, system="DP", model=None, num_total_nodes=None,
                 shuffle_with_dst=False, debug_info=None, replace=True, rng_seed=None):
        if system != "DP":
            raise NotImplementedError(f"system {system!r} needs other GPUs; only 'DP' is available")
        self.rank, self.world_size = rank, world_size
        self.fanouts = list(fanouts)
        self.num_layers = len(self.fanouts)
        self.system = system
        self.replace = replace
        self.rng_seed = rng_seed
        self.batches = 0

    def sample(self, graph, seeds):
        output_nodes = seeds
        blocks = []
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
