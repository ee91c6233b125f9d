"""Captured decode steps: a step of single tokens is launch bound (about nine kernels a layer), so it is
recorded once per (batch size, context length) bucket as a HIP graph and replayed.

The reference records a decode step once and replays it with only the position patched
(docs/08-metal-backend.md:170, docs/24-paged-kv-cache.md:328-334). Here every per-step value lives in one
fixed device buffer (token ids, positions, slots, block tables) that a pinned host buffer is copied into
before each replay; the kernels' launch shapes are those of the bucket, and rows beyond the live batch read
one key of page 0 and store nothing. Nothing that records a memset is captured: buffers are cleared, where
they must be, by fill kernels.
"""
from __future__ import annotations

import gc
from typing import Dict, Sequence, Tuple

import numpy as np
import torch

from ..kernels import ops
from .step import StepEntry


def _bucket(n: int, steps: Sequence[int]) -> int:
    for s in steps:
        if n <= s:
            return s
    return 0


def batch_buckets(max_batch: int):
    """The batch sizes steps are captured at: the powers of two below ``max_batch``, then ``max_batch`` itself, so
    that a full batch is always taken."""
    max_batch = max(int(max_batch), 1)
    sizes = []
    b = 1
    while b < max_batch:
        sizes.append(b)
        b *= 2
    return sizes + [max_batch]


class DecodeGraphs:
    def __init__(self, runner, max_batch: int, context_step: int = 2048, max_graphs: int = 16):
        self.runner = runner
        self.max_graphs = max(1, max_graphs)  # each graph has a memory pool of its own (logits, activations, scratch)
        self.batch_buckets = batch_buckets(max_batch)
        self.context_step = context_step
        self.graphs: Dict[Tuple[int, int], dict] = {}
        self.replays = 0
        self.evictions = 0

    def takes(self, entries: Sequence[StepEntry]) -> bool:
        if not entries or any(len(e.tokens) != 1 for e in entries):
            return False
        if not getattr(self.runner.model, "capturable", True):
            return False
        return _bucket(len(entries), self.batch_buckets) > 0

    def _key(self, entries) -> Tuple[int, int]:
        cache = self.runner.cache
        longest = max(cache.length(e.rid) for e in entries) + 1
        ctx = min(-(-longest // self.context_step) * self.context_step, max(self.runner.max_positions, longest))
        return _bucket(len(entries), self.batch_buckets), ctx

    def run(self, entries: Sequence[StepEntry], feed=None) -> torch.Tensor:
        """The cache already has room for the entries' tokens; returns fp32 logits, one row per entry. ``feed``: the
        entries' tokens as an int32 tensor on the device (the token ids open the step's buffer)."""
        r = self.runner
        bk, ck = self._key(entries)
        width = -(-ck // r.cache.page_size)
        parts, sizes, segments = r._layout(entries, pad_rows=bk, width=width)
        flat = np.concatenate(parts)
        g = self.graphs.pop((bk, ck), None)
        if g is None:
            while len(self.graphs) >= self.max_graphs:  # the one used longest ago goes, with its memory pool
                self._evict(next(iter(self.graphs)))
            g = self._capture(bk, ck, flat, sizes, segments)
        self.graphs[(bk, ck)] = g  # dicts keep insertion order: the last one used is the last one
        g["copied"].synchronize()  # the previous upload out of the pinned buffer has finished
        g["host"].numpy()[:] = flat
        ops.copy_words(g["host"], g["dev"])  # a kernel in the stream, reading the pinned buffer
        g["copied"].record()
        if feed is not None:
            g["dev"][:len(entries)].copy_(feed[:len(entries)])
        g["graph"].replay()
        self.replays += 1
        want = [i for i, e in enumerate(entries) if len(e.want)]
        out = g["logits"]
        if len(want) == len(entries):
            return out[:len(entries)]
        return out[torch.tensor(want, dtype=torch.long, device=out.device)] if want else out[:0]

    def _evict(self, key) -> None:
        """Drops a captured step. Its last replay and the upload kernel that reads its pinned buffer may still be
        queued, and neither the graph's memory pool nor the pinned block may go back to their allocators before
        they have run: the allocators know nothing of kernels that read host memory."""
        g = self.graphs.pop(key)
        g["copied"].synchronize()
        torch.cuda.current_stream().synchronize()
        self.evictions += 1
        del g

    def _capture(self, bk: int, ck: int, flat, sizes, segments) -> dict:
        r = self.runner
        host = torch.empty(flat.shape[0], dtype=torch.int32).pin_memory()
        host.numpy()[:] = flat
        dev = torch.empty(flat.shape[0], dtype=torch.int32, device=r.device)
        dev.copy_(host)
        sizes = dict(sizes)
        sizes["max_context"] = ck  # launch shapes of the bucket, whatever the live requests hold
        ctx = r._context(dev, sizes, segments)
        ctx.segments = []  # a captured step must not depend on host-side facts of one batch
        # once eagerly, so that nothing is loaded or configured for the first time inside the capture
        r.model.forward(ctx, r.cache.slots)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        # No garbage collection while the stream is capturing: an object with a graph, an event or pinned memory of its
        # own (an engine that was dropped earlier, still held by a cycle) must not be destroyed then, since the calls
        # that destroy it are not allowed during a capture and end the process when they fail in a destructor. (No
        # collection in front of the capture either: a full one takes 20 ms with torch loaded, two thirds of what a
        # capture then costs, and a first short completion waits for it.)
        collecting = gc.isenabled()
        gc.disable()
        try:
            with torch.cuda.graph(graph):
                logits = r.model.forward(ctx, r.cache.slots)
        finally:
            if collecting:
                gc.enable()
        torch.cuda.synchronize()
        copied = torch.cuda.Event()
        copied.record()
        return {"graph": graph, "host": host, "dev": dev, "logits": logits, "ctx": ctx, "copied": copied}
