"""Decode steps replayed from HIP graphs.

A decode step of a 36-layer model is some four hundred small launches; issued
one by one from the host they take several times longer than the kernels run.
For steps that feed one token per request the whole forward pass is captured
once per (batch size, block-table width) and replayed: the host then only
fills the step's index arrays into a pinned buffer, copies them to the fixed
device buffer the graph reads, and launches the graph.

The reference does the same with CUDA graphs, one per batch size up to 32,
with fixed input buffers refreshed before each replay
(crates/prelude-cuda/src/cuda_graph.rs:45-332, buffers.rs:11-30).  Here the
block-table width is part of the key (rounded up, so few graphs cover all
context lengths) and graphs are captured when first needed.  At most
``cache_size`` graphs are kept: each owns its logits tensor [B, vocab], so
the number is part of the memory the engine sets aside; when one more is
needed the least recently used is dropped (after the device has finished
with it) and captured again if its shape comes back.

A graph may be launched again while its previous launch still runs (the host
prepares one step ahead): launches on one stream run in order, and the index
buffer is refreshed by a copy on that same stream.

Nothing inside a captured step may depend on the step's data through the
host: launch shapes follow the batch size and the table width only (the
decode attention kernel is launched for as many splits as the table could
hold; workgroups beyond a sequence's length leave at once).
"""
from __future__ import annotations

import collections
import dataclasses
from typing import Sequence, Tuple

import torch


@dataclasses.dataclass
class _Captured:
    graph: torch.cuda.CUDAGraph
    buffer: torch.Tensor      # the fixed int32 index buffer
    logits: torch.Tensor      # the graph's output [B, vocab] float32
    stride: int


class DecodeGraphs:

    def __init__(self, engine, max_batch: int, cache_size: int = 32):
        self.engine = engine
        self.max_batch = int(max_batch)
        self.cache_size = max(1, int(cache_size))
        self._graphs: "collections.OrderedDict[Tuple[int, int], _Captured]" = collections.OrderedDict()
        self._pool = None
        self.replays = 0
        self.captures = 0
        self.evictions = 0

    def eligible(self, entries: Sequence) -> bool:
        if not 1 <= len(entries) <= self.max_batch:
            return False
        return all(len(e.tokens) == 1 and len(e.want) == 1 and int(e.want[0]) == 0 for e in entries)

    def owns(self, t: torch.Tensor) -> bool:
        return any(t is g.logits for g in self._graphs.values())

    def _stride_for(self, ends: Sequence[int]) -> int:
        # the bound the decode kernels round a step's longest context to anyway: a replayed step is then launched
        # exactly as the same step run directly would be
        from ..ops import kernels as K
        page = self.engine.page_size
        return K.decode_context_bound(max(ends), page) // page

    def run(self, entries: Sequence, starts: Sequence[int], carried=None) -> torch.Tensor:
        eng = self.engine
        n = len(entries)
        stride = self._stride_for([s + 1 for s in starts])
        key = (n, stride)
        cap = self._graphs.get(key)
        if cap is None:
            while len(self._graphs) >= self.cache_size:
                # the device may still be replaying it (the host runs a step ahead): wait, then let it go
                torch.cuda.synchronize(eng.device)
                self._graphs.popitem(last=False)
                self.evictions += 1
            cap = self._capture(entries, starts, stride, carried)
            self._graphs[key] = cap
        else:
            self._graphs.move_to_end(key)
            eng.build_batch(entries, starts, stride=stride, device_buffer=cap.buffer, carried=carried)
        cap.graph.replay()
        self.replays += 1
        return cap.logits

    def _capture(self, entries: Sequence, starts: Sequence[int], stride: int, carried=None) -> _Captured:
        eng = self.engine
        n = len(entries)
        size = eng.tables.step_layout(n, n, stride, n)["_total"][1]
        buffer = torch.empty(size, dtype=torch.int32, device=eng.device)
        batch = eng.build_batch(entries, starts, stride=stride, device_buffer=buffer, carried=carried)
        # once outside a capture, on a side stream, so that whatever libraries set up lazily exists already;
        # it writes the same keys and values the replay will write.  State of fixed size is not written twice to
        # the same effect (a recurrence would advance two steps): the slots' rows are put back afterwards.
        stateful = [c for c in eng.caches if hasattr(c, "snapshot")] if eng.model.needs_state else []
        saved = [c.snapshot(batch.state_slots) for c in stateful]
        side = torch.cuda.Stream(device=eng.device)
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            eng.forward(batch)
        torch.cuda.current_stream().wait_stream(side)
        for c, rows in zip(stateful, saved):
            c.restore(batch.state_slots, rows)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        if self._pool is None:
            self._pool = torch.cuda.graph_pool_handle()
        with torch.cuda.graph(graph, pool=self._pool):
            logits = eng.forward(batch)
        self.captures += 1
        return _Captured(graph, buffer, logits, stride)
