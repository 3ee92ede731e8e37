"""Strategy cost model (reference python/npc/cost_model/estimator.py) and the
dry run that feeds it (AllPSNeighborSampler, python/npc/sampler.py:367-600).

The reference runs the dry run on all GPUs of a job, every rank sampling the
whole graph through UVA and exchanging ids with its peers.  Here one GPU that
holds the whole graph plays the world_size ranks in turn: each rank's local work
(sampling, relabel, owner bucketing, virtual-node mapping) runs through this
library's kernels, and the id exchanges between ranks become slices and
concatenations in device memory.  What the cost model consumes is the same: per
strategy and rank the nodes whose features would be loaded, and the send /
receive sizes of the hidden-feature reshuffle.

Strategies, with the reference's internal names: DP (data parallel), NP (the
owner of a last-hop frontier node samples it), SP (sources are replaced by one
virtual node per (owner, destination)), MP (every rank loads a column slice of
all ranks' input nodes).
"""
import time
from dataclasses import dataclass, field
from typing import List, Optional, Sequence

import torch

from . import capi

# MB/s, the reference's measured constants (estimator.py:15-19); pass others for other machines
BYTES_PER_ELEMENT = 4
BW_PCIE = 5594.79
BW_GPU = 5782.60
BW_NETWORK = 4616.41
BW_PURE_NETWORK = 3831.46

STRATEGIES = ("DP", "NP", "SP", "MP")
SYSTEM_NAMES = {"DP": "GDP", "NP": "DNP", "SP": "SNP", "MP": "NFP"}   # estimator.py:689-690
SP_BASE = 10000000                                                       # sampler.py:384


# ---------------------------------------------------------------- arithmetic

def get_cache_miss(seeds_freq, num_cache_nodes, input_dim, made_seeds_freq=None):
    """Feature elements loaded past a cache of the num_cache_nodes most frequent
    nodes of made_seeds_freq (estimator.py:22-30)."""
    ranked = seeds_freq if made_seeds_freq is None else made_seeds_freq
    k = min(int(num_cache_nodes), seeds_freq.numel())
    top = torch.sort(ranked, descending=True, stable=True)[1][:k]
    return (seeds_freq.sum() - seeds_freq[top].sum()) * input_dim


def cachemiss_vol_to_time(vol, bytes_per_element=BYTES_PER_ELEMENT, bw=BW_PCIE):
    """estimator.py:118-119"""
    return vol * bytes_per_element / (1024 * 1024 * bw)


def cpu_cachemiss_vol_to_time(vol, bytes_per_element=BYTES_PER_ELEMENT, bw=BW_PURE_NETWORK):
    """estimator.py:114-115"""
    return vol * bytes_per_element / (1024 * 1024 * bw)


def reshuffle_vol_to_time(vol, multi_machine=True, bytes_per_element=BYTES_PER_ELEMENT):
    """estimator.py:122-124.  The reference tests `args.nproc_per_node`, which is
    -1 on one machine and therefore true either way: BW_NETWORK is what it uses."""
    bw = BW_NETWORK if multi_machine else BW_PCIE
    return vol * bytes_per_element / (1024 * 1024 * bw)


def get_featload_time(seeds_freq, num_gpu_cache_nodes, input_dim, gpu_sorted_idx=None):
    """Single-machine branch of estimator.py:53-71: time to load what misses a
    cache of the first num_gpu_cache_nodes ids of gpu_sorted_idx."""
    if gpu_sorted_idx is None:
        gpu_sorted_idx = torch.sort(seeds_freq, descending=True, stable=True)[1]
    k = min(int(num_gpu_cache_nodes), seeds_freq.numel())
    miss = seeds_freq.sum() - seeds_freq[gpu_sorted_idx[:k]].sum()
    return cachemiss_vol_to_time(miss * input_dim)


def get_reshuffle_dim(model, num_hidden, num_heads=1):
    """estimator.py:127-128"""
    return num_hidden if model != "GAT" else num_hidden * num_heads


def get_dp_reshuffle_vol():
    return 0


def _offset_volume(rank, world_size, offset):
    """Total of an inclusive cumulative offset list without the rank's own bucket."""
    offset = [int(x) for x in offset]
    return offset[world_size - 1] - offset[rank] + (offset[rank - 1] if rank > 0 else 0)


def get_np_reshuffle_vol(rank, world_size, dim, send_offset, recv_offset):
    """estimator.py:135-151: rows sent to and received from the other ranks, forward and backward."""
    return 2 * dim * (_offset_volume(rank, world_size, send_offset) + _offset_volume(rank, world_size, recv_offset))


def get_sp_reshuffle_vol(rank, world_size, dim, send_sizes, recv_sizes, model="SAGE", shuffle_with_dst=False):
    """estimator.py:154-187.  GAT exchanges source rows like NP; the others exchange
    one row per virtual node (and per destination when shuffle_with_dst)."""
    if model == "GAT":
        return get_np_reshuffle_vol(rank, world_size, dim, send_sizes, recv_sizes)
    send_sizes = [int(x) for x in send_sizes]
    recv_sizes = [int(x) for x in recv_sizes]
    vol = 0
    for r in range(world_size):
        if r == rank:
            continue
        if shuffle_with_dst:
            vol += 2 * dim * (send_sizes[3 * r] + send_sizes[3 * r + 2] + recv_sizes[3 * r] + recv_sizes[3 * r + 2])
        else:
            vol += 2 * dim * (send_sizes[2 * r + 1] + recv_sizes[2 * r + 1])
    return vol


def get_mp_reshuffle_vol(world_size, dim, send_size, recv_size):
    """estimator.py:190-197"""
    return 2 * dim * (int(send_size) * (world_size - 2) + sum(int(x) for x in recv_size))


def pick_strategy(costs):
    """costs: {strategy: [sampling, cache miss..., reshuffle]} -> the strategy with
    the smallest total, first of STRATEGIES on ties (np.argmin, estimator.py:691-693)."""
    totals = [float(sum(costs[s])) for s in STRATEGIES]
    return STRATEGIES[min(range(len(STRATEGIES)), key=lambda i: (totals[i], i))]


# ---------------------------------------------------------------- dry run

@dataclass
class RankSample:
    """What AllPSNeighborSampler.sample returns on one rank (sampler.py:593-598)."""
    dp_seeds: torch.Tensor
    np_seeds: torch.Tensor
    np_send_offset: List[int]
    np_recv_offset: List[int]
    sp_seeds: torch.Tensor
    sp_send_sizes: List[int]
    sp_recv_sizes: List[int]
    mp_seeds: torch.Tensor
    mp_send_size: int
    mp_recv_size: List[int]
    # the rank's last-hop frontier and its sampled neighbours (fixed stride, -1 = none)
    frontier: Optional[torch.Tensor] = field(default=None, repr=False)
    neighbors: Optional[torch.Tensor] = field(default=None, repr=False)


def _cumsum(xs):
    out, acc = [], 0
    for x in xs:
        acc += int(x)
        out.append(acc)
    return out


def sp_send_sizes(world_size, num_dst, sorted_nodes, unique_frontier, shuffle_with_dst=False):
    """Local half of SPSampleAndShuffle (src/sampling.cc:71-107): boundaries of the
    owners in the sorted virtual nodes -> sizes in the all-to-all's order, per peer
    (ids sent, virtual nodes) or (destinations, ids, virtual nodes).
    -> (send_sizes list, send_offset list)."""
    per = 3 if shuffle_with_dst else 2
    off = capi.vir_send_offset(world_size, num_dst, sorted_nodes, unique_frontier, shuffle_with_dst).tolist()
    sizes = [off[i + 1] - off[i] for i in range(len(off) - 1)]
    sizes[(per - 1) * world_size] = off[(per - 1) * world_size + 1]
    return [sizes[i * world_size + r] for r in range(world_size) for i in range(per)], off


class AllPSDryRun:
    """All four strategies' view of the same mini-batches, for world_size ranks
    played by one GPU.  fanouts are listed k-hop ... 1-hop and walked in reverse
    as in the reference.  min_vids [world_size + 1] are the owners' id ranges."""

    def __init__(self, graph, world_size, fanouts, min_vids, model="SAGE", num_total_nodes=None,
                 shuffle_with_dst=False, replace=True, rng_seed=0, keep_samples=False):
        self.graph = graph
        self.world_size = int(world_size)
        self.fanouts = list(fanouts)
        self.num_layers = len(self.fanouts)
        self.model = model
        self.shuffle_with_dst = bool(shuffle_with_dst)
        self.min_vids = min_vids.to(graph.device, torch.int64)
        self.num_total_nodes = int(num_total_nodes if num_total_nodes is not None else min_vids[-1])
        self.replace = replace
        self.rng_seed = int(rng_seed)
        self.keep_samples = keep_samples
        self.clear_time_list()

    # the reference's bookkeeping (sampler.py:389-400)
    def get_time_list(self):
        return self.num_sample_times, self.sampling_algo_time, self.time_list

    def clear_time_list(self):
        self.num_sample_times = 0
        self.time_list = [0.0, 0.0, 0.0, 0.0]
        self.sampling_algo_time = [0.0 for _ in range(self.num_layers)]

    def _clock(self):
        torch.cuda.synchronize(self.graph.device)
        return time.perf_counter()

    def _sample(self, rank, frontier, fanout, hop):
        key = self.rng_seed + 0x9E3779B1 * (self.num_sample_times * self.world_size + rank)
        return capi.sample_neighbors(self.graph, frontier, fanout, self.replace, key, hop, want_counts=False)[0]

    def _owner_buckets(self, rank, ids):
        """ShuffleSeeds' local half (src/sampling.cc:159-175) -> (sizes list, ids grouped by owner)."""
        size, _, grouped, _ = capi.cluster_permute(ids, self.min_vids, self.world_size, rank=rank)
        return size.tolist(), grouped

    @staticmethod
    def _route(sizes, grouped):
        """The all-to-all of ShuffleSeeds for every rank at once: sizes[r][q] ids of
        grouped[r] go to rank q -> per receiver (ids in sender order, sizes by sender)."""
        world = len(sizes)
        parts = [torch.split(grouped[r], sizes[r]) for r in range(world)]
        return ([torch.cat([parts[r][q] for r in range(world)]) for q in range(world)],
                [[sizes[r][q] for r in range(world)] for q in range(world)])

    def sample(self, seeds_per_rank: Sequence[torch.Tensor]) -> List[RankSample]:
        """One step of every rank; seeds_per_rank[r] are rank r's seeds (device int64)."""
        W = self.world_size
        if len(seeds_per_rank) != W:
            raise ValueError(f"{len(seeds_per_rank)} seed tensors for world_size {W}")
        self.num_sample_times += 1
        frontier = [capi._dev_i64(s, "seeds") for s in seeds_per_rank]
        hop_fanouts = list(reversed(self.fanouts))
        for hop, fanout in enumerate(hop_fanouts[:-1]):
            t0 = self._clock()
            for r in range(W):
                nbr = self._sample(r, frontier[r], fanout, hop)
                frontier[r] = capi.relabel(frontier[r], nbr)[0]
            self.sampling_algo_time[hop] += (self._clock() - t0) / W
        hop, fanout = self.num_layers - 1, hop_fanouts[-1]

        # NP: the owner samples; it sees each of its frontier nodes once
        t0 = self._clock()
        np_sizes, np_grouped = zip(*(self._owner_buckets(r, frontier[r]) for r in range(W)))
        np_recv, np_recv_sizes = self._route(list(np_sizes), list(np_grouped))
        np_seeds = []
        for q in range(W):
            mine = torch.unique(np_recv[q], sorted=True)
            np_seeds.append(capi.relabel(mine, self._sample(q, mine, fanout, hop))[0])
        self.time_list[1] += (self._clock() - t0) / W

        t0 = self._clock()
        neighbors = [self._sample(r, frontier[r], fanout, hop) for r in range(W)]
        self.sampling_algo_time[hop] += (self._clock() - t0) / W

        # DP (and the frontier MP broadcasts): the block of the local sample
        t0 = self._clock()
        dp_seeds = [capi.relabel(frontier[r], neighbors[r])[0] for r in range(W)]
        dp_time = (self._clock() - t0) / W
        self.time_list[0] += dp_time

        t0 = self._clock()
        sp = self._sp_gat(frontier, neighbors) if self.model == "GAT" else self._sp(frontier, neighbors, fanout)
        self.time_list[2] += (self._clock() - t0) / W

        # MP: everyone receives everyone's input nodes (MPSampleShuffle, src/sampling.cc:195-245)
        t0 = self._clock()
        mp_seeds = torch.cat(dp_seeds)
        if self.model == "GAT":
            mp_send = [int(d.numel()) for d in dp_seeds]
        else:
            mp_send = [int(f.numel()) for f in frontier]
        self.time_list[3] += (self._clock() - t0) / W + dp_time    # MP relabels the same block first

        out = []
        for r in range(W):
            out.append(RankSample(
                dp_seeds=dp_seeds[r],
                np_seeds=np_seeds[r], np_send_offset=_cumsum(np_sizes[r]), np_recv_offset=_cumsum(np_recv_sizes[r]),
                sp_seeds=sp[r][0], sp_send_sizes=sp[r][1], sp_recv_sizes=sp[r][2],
                mp_seeds=mp_seeds, mp_send_size=mp_send[r], mp_recv_size=list(mp_send),
                frontier=frontier[r] if self.keep_samples else None,
                neighbors=neighbors[r] if self.keep_samples else None))
        return out

    def _sp_gat(self, frontier, neighbors):
        """sampler.py:444-466: the distinct sources go to their owners (ShuffleSeeds)."""
        W = self.world_size
        sizes, grouped = [], []
        for r in range(W):
            src = torch.unique(neighbors[r][neighbors[r] >= 0], sorted=True)
            ids = torch.cat((frontier[r], src)) if self.shuffle_with_dst else src
            s, g = self._owner_buckets(r, ids)
            sizes.append(s)
            grouped.append(g)
        recv, recv_sizes = self._route(sizes, grouped)
        return [(recv[q] if self.shuffle_with_dst else torch.cat((frontier[q], recv[q])),
                 _cumsum(sizes[q]), _cumsum(recv_sizes[q])) for q in range(W)]

    def _sp(self, frontier, neighbors, fanout):
        """sampler.py:467-557: sources -> virtual nodes (owner, destination); the
        owner receives the source ids of its virtual nodes (and, with
        shuffle_with_dst, the destinations it owns)."""
        W, per = self.world_size, 3 if self.shuffle_with_dst else 2
        send_sizes, to_owner_src, to_owner_dst = [], [], []
        for r in range(W):
            dst, src = frontier[r], neighbors[r]
            nd = dst.numel()
            valid = src >= 0
            if self.shuffle_with_dst:
                vir = capi.map_to_vir(src, fanout, self.min_vids, W, rank=r, dst=dst)
                keep = torch.cat((torch.ones(nd, dtype=torch.bool, device=dst.device), valid))
                ids = torch.cat((dst, src))
            else:
                vir = capi.map_to_vir(src, fanout, self.min_vids, W, rank=r, num_dst=nd)
                keep, ids = valid, src
            vir, ids = vir[keep], ids[keep]
            sorted_vir, perm = torch.sort(vir, stable=True)
            ids = ids[perm]
            lead = nd if self.shuffle_with_dst else 0
            unique_frontier = torch.unique(sorted_vir[lead:], sorted=True)
            sizes, off = sp_send_sizes(W, nd, sorted_vir, unique_frontier, self.shuffle_with_dst)
            send_sizes.append(sizes)
            if self.shuffle_with_dst:
                to_owner_dst.append([ids[off[q]:off[q + 1]] for q in range(W)])
                to_owner_src.append([ids[off[W + q]:off[W + q + 1]] for q in range(W)])
            else:
                to_owner_src.append([ids[off[q]:off[q + 1]] for q in range(W)])
        out = []
        for q in range(W):
            recv_sizes = [send_sizes[r][per * q + i] for r in range(W) for i in range(per)]
            unique_src = torch.unique(torch.cat([to_owner_src[r][q] for r in range(W)]), sorted=True)
            if self.shuffle_with_dst:
                seeds = torch.cat([to_owner_dst[r][q] for r in range(W)] + [unique_src])
            elif self.model == "GCN":
                seeds = unique_src
            else:
                seeds = torch.cat((frontier[q], unique_src))
            out.append((seeds, send_sizes[q], recv_sizes))
        return out


@dataclass
class StrategyCosts:
    """Seconds per step and strategy: [sampling, feature loading, reshuffle]."""
    costs: dict
    best: str

    @property
    def best_system(self):
        return SYSTEM_NAMES[self.best]


def estimate(dryrun: AllPSDryRun, batches_per_rank, rank=0, *, input_dim, num_hidden, num_heads=1,
             cache_memory=0, mp_input_dim=None, gpu_sorted_idx=None):
    """The single-machine cost model of run_costmodel (estimator.py:392-693) for one
    rank: access frequencies of each strategy's input nodes -> cache-miss time for a
    cache of cache_memory bytes (ranked by gpu_sorted_idx[strategy], or by the
    strategy's own frequency), reshuffle volume -> time, measured sampling time.
    batches_per_rank: iterable of per-step seed lists (one tensor per rank)."""
    W, model = dryrun.world_size, dryrun.model
    dim = get_reshuffle_dim(model, num_hidden, num_heads)
    dev = dryrun.graph.device
    freq = {s: torch.zeros(dryrun.num_total_nodes, dtype=torch.int64, device=dev) for s in STRATEGIES}
    vol = {s: 0 for s in STRATEGIES}
    dryrun.clear_time_list()
    steps = 0
    for seeds_per_rank in batches_per_rank:
        res = dryrun.sample(seeds_per_rank)[rank]
        steps += 1
        for s, ids in (("DP", res.dp_seeds), ("NP", res.np_seeds), ("SP", res.sp_seeds), ("MP", res.mp_seeds)):
            capi.count_ids(ids, freq[s])
        vol["NP"] += get_np_reshuffle_vol(rank, W, dim, res.np_send_offset, res.np_recv_offset)
        vol["SP"] += get_sp_reshuffle_vol(rank, W, dim, res.sp_send_sizes, res.sp_recv_sizes, model,
                                          dryrun.shuffle_with_dst)
        vol["MP"] += get_mp_reshuffle_vol(W, dim, res.mp_send_size, res.mp_recv_size)
    if steps == 0:
        raise ValueError("estimate: no batches")
    _, algo, other = dryrun.get_time_list()
    sampling = {"DP": sum(algo) + other[0], "NP": sum(algo[:-1]) + other[1],
                "SP": sum(algo) + other[2], "MP": sum(algo) + other[3]}
    cache_nodes = int(cache_memory / (input_dim * BYTES_PER_ELEMENT))
    mp_dim = mp_input_dim if mp_input_dim is not None else -(-input_dim // W)
    ranked = gpu_sorted_idx or {}
    costs = {}
    for s in STRATEGIES:
        nodes, d = (cache_nodes * W, mp_dim) if s == "MP" else (cache_nodes, input_dim)
        load = float(get_featload_time(freq[s], nodes, d, ranked.get(s)))
        costs[s] = [sampling[s] / steps, load / steps, reshuffle_vol_to_time(vol[s]) / steps]
    return StrategyCosts(costs, pick_strategy(costs))
