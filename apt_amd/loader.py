"""Epoch loader: what `dgl.dataloading.DataLoader(graph, indices, graph_sampler,
batch_size, shuffle, drop_last)` does around the sampler in the reference's
trainer (examples/train.py:84-94), with several mini-batches in flight.

Hops 1 and 2 of a batch are strings of short kernels that leave most of the GPU
idle, the last hop is bound by random memory transactions and the gather by
bandwidth, so batches on different streams overlap well: `in_flight` pipelines
(own buffers and rank table each) run on streams of their own, and the consumer
receives batch i while batches i+1 .. i+in_flight-1 are being built.

The per-batch host work (a dozen kernel launches, the copy of the sizes, the
events) is done by a thread of the C library (apt_epoch_*, capi.EpochDriver):
the Python thread only waits for the next batch and narrows its buffers, block
formats (COO / CSC / CSR) included.  With graph replay requested the batches are
enqueued from Python instead (driver="python" forces that path).
"""
import torch

from .pipeline import MiniBatchPipeline


class MiniBatchLoader:
    def __init__(self, graph, feat, indices, batch_size, hop_fanouts, in_flight=4, shuffle=True, drop_last=True,
                 replace=False, seed=0, formats=False, requests=None, use_graph=False, as_blocks=False,
                 driver="auto", streams=None):
        """indices: node ids to draw seeds from (the training ids).  hop_fanouts
        start from the seeds.  Yields MiniBatchPipeline.result() dicts with
        `output_nodes` (the batch's seeds) added.  A yielded batch lives in its
        pipeline's buffers: it stays valid until the loader is asked for the next
        one, and work the consumer has enqueued on its current stream by then is
        waited for before the buffers are reused.  use_graph: every pipeline
        replays a captured HIP graph, which costs the host less per batch (worth it
        for small batches, where the host's launch calls are the limit).  as_blocks:
        batch["blocks"] are sampler.Block objects, ready for apt_amd.layers.
        formats: as MiniBatchPipeline's (True / "inner" / "csc": the blocks also in COO + CSC, with CSR for all /
        all but the outermost / none).
        driver: "c" = batches are enqueued by the C library's epoch thread (not with use_graph),
        "python" = from this thread, "auto" = "c" where it applies.
        streams: the torch.cuda.Stream objects to build batches on, one per batch in flight (default: new ones;
        never the consumer's stream).  A process has few hardware queues (HIP's GPU_MAX_HW_QUEUES, 4 by default) and
        its streams are dealt onto them as they are created, so in a process that has created other streams two of
        the loader's may share a queue and take turns; a caller that knows better passes its own."""
        if in_flight < 1:
            raise ValueError("in_flight must be >= 1")
        dev = graph.device
        self.device = dev
        self.indices = indices.to(dev, torch.int64)
        self.batch_size = int(batch_size)
        self.shuffle, self.drop_last, self.seed = bool(shuffle), bool(drop_last), int(seed)
        n = self.indices.numel()
        self.num_full = n // self.batch_size
        self.tail = 0 if drop_last else n - self.num_full * self.batch_size
        if self.num_full + (1 if self.tail else 0) == 0:
            raise ValueError(f"{n} indices give no batch of {self.batch_size}")
        kw = dict(replace=replace, formats=formats, requests=requests, use_graph=use_graph)
        self._make = lambda b: MiniBatchPipeline(graph, feat, b, hop_fanouts, **kw)
        self.pipes = [self._make(self.batch_size) for _ in range(min(in_flight, max(self.num_full, 1)))]
        if streams is not None:
            streams = list(streams)
            if len(streams) < len(self.pipes):
                raise ValueError(f"{len(streams)} streams for {len(self.pipes)} batches in flight")
            if any(not isinstance(st, torch.cuda.Stream) or st.cuda_stream == 0 for st in streams):
                raise ValueError("streams must be torch.cuda.Stream objects other than the default stream")
        self.streams = streams[:len(self.pipes)] if streams is not None else [torch.cuda.Stream(device=dev) for _ in self.pipes]
        self.done = [torch.cuda.Event() for _ in self.pipes]
        self.released = [torch.cuda.Event() for _ in self.pipes]
        self.tail_pipe = self._make(self.tail) if self.tail else None     # the short last batch has buffers of its own
        self.as_blocks = bool(as_blocks)
        self.epoch = 0
        if driver not in ("auto", "c", "python"):
            raise ValueError("driver must be 'auto', 'c' or 'python'")
        c_ok = not use_graph
        if driver == "c" and not c_ok:
            raise ValueError("the C epoch driver does not replay graphs: use driver='python'")
        from . import capi
        if len(self.pipes) > capi.MAX_SLOTS:
            if driver == "c":
                raise ValueError(f"the C epoch driver takes at most {capi.MAX_SLOTS} batches in flight")
            c_ok = False
        self._c_driver = None
        self._use_c = c_ok and driver != "python"
        # The C driver enqueues batch i + F behind batch i on the same stream without waiting for the consumer,
        # so that no stream runs dry between a batch's completion and the consumer's release of it: that takes a
        # second set of buffers per stream (the two sets of a stream share its rank table).
        self._spare = ([MiniBatchPipeline(graph, feat, self.batch_size, hop_fanouts, table=p.plan.table, **kw)
                        for p in self.pipes] if self._use_c and 2 * len(self.pipes) <= capi.MAX_SLOTS else [])

    def __len__(self):
        return self.num_full + (1 if self.tail else 0)

    def host_cost(self):
        """What the C driver's thread has spent enqueueing and what the consumer has spent waiting, in seconds,
        since the loader's first epoch (capi.EpochDriver.host_cost); None on the Python path."""
        return self._c_driver.host_cost() if self._c_driver is not None else None

    def _launch(self, k, pipe, seeds, rng_seed, after):
        st = self.streams[k]
        st.wait_event(after)
        with torch.cuda.stream(st):
            pipe.run(seeds, rng_seed)
            pipe.stage_sizes()
            self.done[k].record(st)

    def __iter__(self):
        cur = torch.cuda.current_stream(self.device)
        ids = self.indices
        if self.shuffle:
            gen = torch.Generator(device=self.device)
            gen.manual_seed(self.seed * 1000003 + self.epoch)
            ids = ids[torch.randperm(ids.numel(), generator=gen, device=self.device)]
        full = ids[:self.num_full * self.batch_size].view(self.num_full, self.batch_size)
        batches = [full[i] for i in range(self.num_full)]
        if self.tail:
            batches.append(ids[self.num_full * self.batch_size:])
        rng0 = (self.seed * 7919 + self.epoch) * len(self)
        self.epoch += 1
        F = len(self.pipes)
        ready = torch.cuda.Event()
        ready.record(cur)                                  # the seeds above were produced on the consumer's stream
        if self._use_c:
            yield from self._iter_c(full, batches, rng0, ready)
            return

        def launch(i, after):
            k = i % F
            pipe = self.tail_pipe if (self.tail and i == len(batches) - 1) else self.pipes[k]
            self._launch(k, pipe, batches[i], rng0 + i, after)
            return pipe

        owner = {}
        for i in range(min(F, len(batches))):
            owner[i] = launch(i, ready)
        for i in range(len(batches)):
            k = i % F
            cur = torch.cuda.current_stream(self.device)
            cur.wait_event(self.done[k])
            self.done[k].synchronize()                     # the sizes are in pinned host memory now
            out = owner.pop(i).result(staged=True, as_blocks=self.as_blocks)
            out["output_nodes"] = batches[i]
            yield out
            if i + F < len(batches):
                # whatever the consumer enqueued on its stream for batch i runs before the buffers are reused
                cur = torch.cuda.current_stream(self.device)
                self.released[k].record(cur)
                owner[i + F] = launch(i + F, self.released[k])

    def _iter_c(self, full, batches, rng0, ready):
        """The epoch through the C library's driver: its thread enqueues batch i on pipeline i % F; this
        thread waits for batches in order.  The short last batch (drop_last=False) has buffers of its own and
        is run from here after the others."""
        from . import capi
        slots = self.pipes + self._spare
        if self._c_driver is None:
            self._c_driver = capi.EpochDriver(slots, (self.streams + self.streams)[:len(slots)])
        drv = self._c_driver
        if self.num_full:
            drv.begin(full.reshape(-1), self.num_full, rng0, ready)
            try:
                for i in range(self.num_full):
                    k, sizes, rs, fe = drv.next()
                    pipe = slots[k]
                    pipe.seeds = batches[i]
                    out = pipe.result(as_blocks=self.as_blocks, sizes=sizes, request_sizes=rs, format_edges=fe)
                    out["output_nodes"] = batches[i]
                    yield out
                    drv.release()
            finally:
                drv.end()
        if self.tail:
            cur = torch.cuda.current_stream(self.device)
            self.released[0].record(cur)
            self._launch(0, self.tail_pipe, batches[-1], rng0 + self.num_full, self.released[0])
            cur.wait_event(self.done[0])
            self.done[0].synchronize()
            out = self.tail_pipe.result(staged=True, as_blocks=self.as_blocks)
            out["output_nodes"] = batches[-1]
            yield out
