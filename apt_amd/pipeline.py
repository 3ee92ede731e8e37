"""Whole mini-batch on the GPU without host round trips.

The reference's driver (python/npc/sampler.py:187-203,358-364 then
python/npc/ops.py:598-600) synchronises the stream after every kernel and reads
the unique count back on every hop.  Here every buffer is allocated once at its
upper bound (hop h holds at most B * prod(1 + f_i) frontier rows), the counts
stay in device memory and are read by the next kernel, and the host waits once
per batch, when it wants the sizes.

Two drivers give identical results:
  fused=True   apt_minibatch_sample: one C call per batch, node-indexed rank
               table for relabel (default);
  fused=False  apt_sample_neighbors + apt_relabel per hop (hash-table relabel).
With use_graph=True the fused batch (and the gather) is captured once into a
HIP graph and replayed; seeds and the rng seed are read from fixed device
buffers that are refreshed before each replay.
"""
import torch

from . import capi


class MiniBatchPipeline:
    def __init__(self, graph, feat, batch_size, hop_fanouts, replace=False, gather=True, fused=True,
                 use_graph=False, requests=None, formats=False, defer_lookup=False, table=None, relabel="hash"):
        """hop_fanouts: fanout per hop starting from the seeds (the reference's
        --fan_out list reversed).

        requests: dict(feat_pos_map, remote_worker_map, min_vids, world_size,
        num_remote_workers) for a partitioned feature store.  The input nodes
        are then bucketed as cluster_reqs does (reference
        src/load_subtensor.cc:41-56,83-86): bucket 0 = rows present on this GPU,
        which are gathered; the other buckets are the per-owner request lists
        that the reference would send (left in `request_ids`, grouped by
        bucket, sizes in `request_sizes`).

        defer_lookup: run() lets the relabel's last pass (slots that lost the race for a node read the winner's id)
        ride in the launch of the gather that follows it instead of launching it before: 3-5 % less time per
        batch, while that launch gets 2-3 us longer (it is no longer the gather alone).  Only where the gather
        is what follows the sampling (fused driver, features gathered, no requests, no formats).

        relabel (per-hop driver, fused=False): "hash" = apt_relabel's hash table per hop; "ranked" =
        apt_relabel_ranked, the per-hop calls through a node-indexed rank table, later hops continuing the batch;
        "ranked_bidding" = the same with the table's bids placed by the sampling call of the hop
        (apt_sample_neighbors_bidding; fanouts up to 64, wider hops fall back to "ranked").

        table: the rank table of another pipeline (fused driver) whose batches run on the same stream as this
        one's: batches that follow each other on one stream can share a table (444 MB at 111 M nodes).

        formats: True, "inner" or "csc" also emits every hop's block as COO + CSC, what DGL derives from
        (row, col) in the reference (python/npc/sampler.py:59-69); result() then carries them per block.
        True adds CSR for every block, "inner" for all but the outermost one (the largest; its CSR serves the
        gradient with respect to the layer's input, which a first layer that aggregates the raw features never
        asks for), "csc" for none."""
        self.graph, self.feat = graph, feat
        self.fanouts = [int(f) for f in hop_fanouts]
        self.replace = bool(replace)
        self.fused = bool(fused)
        dev = graph.device
        self.device = dev
        H = len(self.fanouts)
        i64 = dict(dtype=torch.int64, device=dev)
        if self.fused:
            self.plan = capi.MinibatchPlan(graph, batch_size, self.fanouts, replace=replace, table=table)
            self.caps = self.plan.caps
            self.sizes = self.plan.sizes
            self.neighbors, self.relabeled, self.counts = (self.plan.neighbors, self.plan.relabeled,
                                                           self.plan.counts)
            self.nodes = self.plan.nodes
        else:
            self.caps = [int(batch_size)]
            for f in self.fanouts:
                self.caps.append(self.caps[-1] * (1 + f))
            self.neighbors = [torch.empty(self.caps[h] * f, **i64) for h, f in enumerate(self.fanouts)]
            self.relabeled = [torch.empty(self.caps[h] * f, **i64) for h, f in enumerate(self.fanouts)]
            self.counts = [torch.empty(self.caps[h], **i64) for h in range(H)]
            self.frontier = [None] + [torch.empty(self.caps[h + 1], **i64) for h in range(H)]
            # sizes[h] = rows of the frontier entering hop h; sizes[H] = input nodes; then edges
            self.sizes = torch.zeros(H + 2, **i64)
            if relabel not in ("hash", "ranked", "ranked_bidding"):
                raise ValueError("relabel must be 'hash', 'ranked' or 'ranked_bidding'")
            self.ranked = capi.RankedRelabel(graph.num_total_nodes, dev) if relabel != "hash" else None
            self.bid_in_sampler = relabel == "ranked_bidding"
            self.ranked_outside = torch.zeros(1, **i64)    # ids the rank table cannot hold (stays 0 for a valid graph)
            self.workspace = torch.empty(capi.relabel_workspace_bytes(self.caps[-1]), dtype=torch.uint8,
                                         device=dev)
        self.features = None
        if gather and feat is not None:
            self.features = torch.empty((self.caps[-1], feat.out_dim), dtype=feat.dtype, device=dev)
        self.misses = torch.zeros(1, **i64)
        self.requests = requests
        if requests is not None:
            R = int(requests["num_remote_workers"])
            self.request_sizes = torch.zeros(R, **i64)
            self.request_offsets = torch.zeros(R, **i64)
            self.request_ids = torch.empty(self.caps[-1], **i64)
            self.request_perm = torch.empty(self.caps[-1], **i64)
            need = int(capi.lib().apt_bucket_workspace_bytes(self.caps[-1], R))
            self.request_ws = torch.empty(need, dtype=torch.uint8, device=dev)
        self.formats = None
        if formats:
            if formats is not True and formats not in ("csc", "inner"):
                raise ValueError("formats must be False, True, 'inner' or 'csc'")
            self.format_edges = torch.zeros(H, **i64)             # edge count of every hop's block, read in one go
            with_csr = lambda h: formats is True or (formats == "inner" and h < H - 1)   # hop H - 1 = the outermost block
            self.formats = [capi.BlockFormats(self.caps[h], f, self.caps[h + 1], want_csr=with_csr(h), device=dev,
                                              num_edges=self.format_edges[h:h + 1])
                            for h, f in enumerate(self.fanouts)]
            # with CSR a hop's formats are a string of ~10 small dependent launches: the hops then run beside
            # each other (and beside the gather) on streams of their own; COO + CSC alone are 2 launches per
            # hop, less than what the cross-stream joins cost, and stay on the caller's stream
            self.format_side_streams = formats != "csc"
            self.format_streams = [torch.cuda.Stream(device=dev) for _ in self.fanouts]
            self.format_fork = torch.cuda.Event()
            self.format_done = [torch.cuda.Event() for _ in self.fanouts]
        # the relabel's last pass can ride in the gather's launch when the gather is what follows the sampling
        self.can_defer_lookup = (bool(defer_lookup) and self.fused and self.features is not None
                                 and requests is None and not formats)
        self.seeds = None
        self.sizes_host = None
        self.format_edges_host = None
        self.graph_exec = None
        if use_graph:
            if not self.fused:
                raise ValueError("graph replay needs the fused driver")
            self._capture()

    # ------------------------------------------------------------ unfused
    def _size(self, h):
        return self.sizes[h:h + 1]

    def _sample_unfused(self, seeds, rng_seed):
        self.frontier[0] = seeds
        self.sizes.zero_()
        self.sizes[0:1].fill_(seeds.numel())
        total = self.sizes[-1:]
        for h, f in enumerate(self.fanouts):
            n_dev = None if h == 0 else self._size(h)
            if self.ranked is not None and self.bid_in_sampler and f <= 64:
                # the sampler places the relabel's bids on the way (what the operators do for the reference's
                # per-hop calls)
                self.ranked.sample_bidding(self.graph, self.frontier[h], f, self.replace, rng_seed, h, h > 0,
                                           self.neighbors[h], self.relabeled[h], num_frontier_dev=n_dev,
                                           out_counts=self.counts[h], out_total=total,
                                           num_outside_dev=self.ranked_outside)
                self.ranked.enqueue(self.frontier[h], self.neighbors[h], h > 0, self.frontier[h + 1], self.relabeled[h],
                                    self._size(h + 1), self.ranked_outside, num_seeds_dev=n_dev, neighbor_stride=f,
                                    bids_placed=True)
                continue
            capi.sample_neighbors(self.graph, self.frontier[h], f, self.replace, rng_seed, h,
                                  num_frontier_dev=n_dev, out_neighbors=self.neighbors[h],
                                  out_counts=self.counts[h], out_total=total)
            if self.ranked is not None:
                self.ranked.enqueue(self.frontier[h], self.neighbors[h], h > 0, self.frontier[h + 1], self.relabeled[h],
                                    self._size(h + 1), self.ranked_outside, num_seeds_dev=n_dev, neighbor_stride=f)
                continue
            capi.relabel(self.frontier[h], self.neighbors[h], num_seeds_dev=n_dev, neighbor_stride=f,
                         unique=self.frontier[h + 1], relabeled=self.relabeled[h],
                         num_unique_dev=self._size(h + 1), workspace=self.workspace, sync=False)

    # ------------------------------------------------------------ graph
    def _capture(self):
        self.static_seeds = torch.zeros(self.caps[0], dtype=torch.int64, device=self.device)
        # run once eagerly so lazy initialisation happens outside the capture
        self.plan.launch(self.static_seeds, rng_seed=None, defer_lookup=self.can_defer_lookup)
        self.emit_formats()
        if self.features is not None:
            self.gather()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            self.plan.launch(self.static_seeds, rng_seed=None, defer_lookup=self.can_defer_lookup)
            self.emit_formats(join=False)
            if self.features is not None:
                self.gather()
            self.join_formats()
        self.graph_exec = g

    # ------------------------------------------------------------ public
    def sample(self, seeds, rng_seed, defer_lookup=False):
        """Sampling + relabel for every hop, asynchronous.
        defer_lookup (fused driver, no requests, no formats): the relabel's last pass, which only the blocks'
        compact ids wait for, is left to ride in the launch of the gather() that must follow."""
        if seeds.numel() != self.caps[0]:
            raise ValueError(f"expected {self.caps[0]} seeds, got {seeds.numel()}")
        self.seeds = seeds
        if self.fused:
            self.plan.launch(seeds, rng_seed, defer_lookup=defer_lookup and self.can_defer_lookup)
        else:
            self._sample_unfused(seeds, rng_seed)

    def emit_formats(self, join=True):
        """COO / CSC / CSR of every hop's block, asynchronous (no-op unless asked
        for).  Each hop is emitted on its own stream once the current stream has
        finished sampling; join=False leaves the current stream free to go on (the
        gather) and the caller joins later with join_formats()."""
        if self.formats is None:
            return
        if not self.format_side_streams:
            for h, fmt in enumerate(self.formats):
                fmt.emit(self.relabeled[h], self._size(h))
            return
        self.format_fork.record()
        for h, fmt in enumerate(self.formats):
            with torch.cuda.stream(self.format_streams[h]):
                self.format_streams[h].wait_event(self.format_fork)
                fmt.emit(self.relabeled[h], self._size(h))
                self.format_done[h].record()
        if join:
            self.join_formats()

    def join_formats(self):
        """The current stream waits for the formats (before the buffers are reused)."""
        if self.formats is not None and self.format_side_streams:
            cur = torch.cuda.current_stream()
            for e in self.format_done:
                cur.wait_event(e)

    def gather(self):
        """Features of the input nodes (the last hop's unique ids), asynchronous."""
        H = len(self.fanouts)
        index = self.nodes if self.fused else self.frontier[H]
        if self.requests is None:
            pending = self.plan.pending if self.fused and self.plan.pending.open else None
            capi.gather_rows(self.feat, index, num_index_dev=self._size(H), out=self.features,
                             miss_count=self.misses, pending=pending)
            return
        rq = self.requests
        capi.cluster_reqs(index, rq["feat_pos_map"], rq["remote_worker_map"], rq["min_vids"],
                          rq["world_size"], rq["num_remote_workers"], n_dev=self._size(H),
                          out=(self.request_sizes, self.request_offsets, self.request_ids,
                               self.request_perm), workspace=self.request_ws)
        # rows that are here: features[k] belongs to request_ids[k], k < request_sizes[0]
        capi.gather_rows(self.feat, self.request_ids, num_index_dev=self.request_sizes[0:1],
                         out=self.features, miss_count=self.misses)

    def run(self, seeds, rng_seed):
        if self.graph_exec is not None:
            self.static_seeds.copy_(seeds)
            self.plan.rng_seed_dev.fill_(int(rng_seed) & 0x7FFFFFFFFFFFFFFF)
            self.seeds = self.static_seeds
            self.graph_exec.replay()
            return
        self.sample(seeds, rng_seed, defer_lookup=True)
        self.emit_formats(join=False)
        if self.features is not None:
            self.gather()
        self.join_formats()

    def stage_sizes(self):
        """Asynchronous copy of the batch's sizes (and request bucket sizes) to pinned
        host memory on the current stream; result(staged=True) reads them once the
        caller has waited for that stream, without a synchronous device read."""
        if self.sizes_host is None:
            self.sizes_host = torch.empty(self.sizes.numel(), dtype=torch.int64, pin_memory=True)
            if self.requests is not None:
                self.request_sizes_host = torch.empty(self.request_sizes.numel(), dtype=torch.int64,
                                                      pin_memory=True)
        self.sizes_host.copy_(self.sizes, non_blocking=True)
        if self.requests is not None:
            self.request_sizes_host.copy_(self.request_sizes, non_blocking=True)
        if self.formats is not None:
            if self.format_edges_host is None:
                self.format_edges_host = torch.empty(len(self.fanouts), dtype=torch.int64, pin_memory=True)
            self.format_edges_host.copy_(self.format_edges, non_blocking=True)

    def result(self, staged=False, as_blocks=False, sizes=None, request_sizes=None, format_edges=None):
        """Waits for the batch and narrows the buffers to their real sizes ->
        dict(input_nodes, blocks (outermost first), features, num_edges).
        staged: the sizes were copied by stage_sizes() and that copy has finished.
        sizes (and request_sizes, format_edges): the batch's sizes as host lists, when the caller already has them
        (the epoch driver reads them from pinned memory); nothing is waited for then.
        as_blocks: the blocks come as sampler.Block objects (what the layers of
        apt_amd.layers take) instead of dicts; they live in this pipeline's buffers
        like everything else, so a training step must finish with them before the
        pipeline runs its next batch."""
        if self.fused and self.plan.pending.open:      # sampled with the last pass deferred and never gathered
            self.plan.pending.run()
        if sizes is None:
            sizes = self.sizes_host.tolist() if staged else self.sizes.cpu().tolist()
        fmt_edges = None
        if self.formats is not None:
            fmt_edges = (format_edges if format_edges is not None else
                         self.format_edges_host.tolist() if staged else self.format_edges.cpu().tolist())
        H = len(self.fanouts)
        blocks = []
        for h, f in enumerate(self.fanouts):
            n = sizes[h]
            if self.fused:
                src = self.seeds if h == 0 else self.nodes[:n]
                uniq = self.nodes[:sizes[h + 1]]
            else:
                src, uniq = self.frontier[h][:n], self.frontier[h + 1][:sizes[h + 1]]
            blocks.insert(0, dict(seeds=src, neighbors=self.neighbors[h][:n * f],
                                  relabeled=self.relabeled[h][:n * f], counts=self.counts[h][:n],
                                  unique=uniq, fanout=f))
            if self.formats is not None:
                blocks[0]["formats"] = self.formats[h].narrow(num_dst=n, num_src=sizes[h + 1], num_edges=fmt_edges[h])
            if as_blocks:
                from .sampler import Block
                b = blocks[0]
                blocks[0] = Block(sizes[h + 1], n, uniq, b["relabeled"], f, b.get("formats"))
        feats = None if self.features is None else self.features[:sizes[H]]
        inp = self.nodes[:sizes[H]] if self.fused else self.frontier[H][:sizes[H]]
        out = dict(input_nodes=inp, blocks=blocks, features=feats, num_edges=sizes[-1],
                   sizes=sizes[:-1])
        if self.requests is not None:
            rs = request_sizes if request_sizes is not None else (
                self.request_sizes_host.tolist() if staged else self.request_sizes.cpu().tolist())
            out.update(request_sizes=rs, request_ids=self.request_ids[:sizes[H]],
                       request_perm=self.request_perm[:sizes[H]],
                       features=None if self.features is None else self.features[:rs[0]])
        return out
