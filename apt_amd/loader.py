"""Epoch loader: what `dgl.dataloading.DataLoader(graph, indices, graph_sampler,
batch_size, shuffle, drop_last)` does around the sampler in the reference's
trainer (examples/train.py:84-94), with several mini-batches in flight.

Hops 1 and 2 of a batch are strings of short kernels that leave most of the GPU
idle, the last hop is bound by random memory transactions and the gather by
bandwidth, so batches on different streams overlap well: `in_flight` pipelines
(own buffers and rank table each) run on streams of their own, and the consumer
receives batch i while batches i+1 .. i+in_flight-1 are being built.
"""
import torch

from .pipeline import MiniBatchPipeline


class MiniBatchLoader:
    def __init__(self, graph, feat, indices, batch_size, hop_fanouts, in_flight=4, shuffle=True, drop_last=True,
                 replace=False, seed=0, formats=False, requests=None, use_graph=False, as_blocks=False):
        """indices: node ids to draw seeds from (the training ids).  hop_fanouts
        start from the seeds.  Yields MiniBatchPipeline.result() dicts with
        `output_nodes` (the batch's seeds) added.  A yielded batch lives in its
        pipeline's buffers: it stays valid until the loader is asked for the next
        one, and work the consumer has enqueued on its current stream by then is
        waited for before the buffers are reused.  use_graph: every pipeline
        replays a captured HIP graph, which costs the host less per batch (worth it
        for small batches, where the host's launch calls are the limit).  as_blocks:
        batch["blocks"] are sampler.Block objects, ready for apt_amd.layers."""
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
        self.streams = [torch.cuda.Stream(device=dev) for _ in self.pipes]
        self.done = [torch.cuda.Event() for _ in self.pipes]
        self.released = [torch.cuda.Event() for _ in self.pipes]
        self.tail_pipe = self._make(self.tail) if self.tail else None     # the short last batch has buffers of its own
        self.as_blocks = bool(as_blocks)
        self.epoch = 0

    def __len__(self):
        return self.num_full + (1 if self.tail else 0)

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
