"""Steps replayed from HIP graphs.

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

Small steps that bring portions of prompts are bound by the host's launches
as well (a 128-token prompt of a 28-layer model is some 280 launches of a few
microseconds of device work each), so they are replayed too, where every part
of the model allows it (``Part.GRAPH_SAFE_PORTIONS``): such a step's key is
its portion lengths, its number of wanted rows, its table width and whether
every portion has at least its own length of context behind it (which decides
how the prefill attention cuts its work).  There are many such shapes and most
come once, so a shape is captured when it is met a second time.  The reference
captures decode steps only.
"""
from __future__ import annotations

import collections
import dataclasses
import gc
import weakref
from typing import Sequence

import torch


# What a step with portions is taken to cost, to tell where its capture pays: the host 8 us for each launch the
# model's parts count for themselves (``Part.LAUNCHES``); the device the weights streamed once at 4 TB/s or, beyond
# a few tokens, two operations per matrix element and token at 0.4 PFLOP/s (what the library's products reach at
# some hundred rows).
HOST_SECONDS_PER_LAUNCH = 8e-6
STREAM_BYTES_PER_SECOND = 4e12
PRODUCT_OPS_PER_SECOND = 0.4e15


def portion_tokens_worth_a_graph(matrix_elements: int, launches: int, element_bytes: int, cap: int) -> int:
    """Up to how many tokens a step with portions is replayed from a graph: as long as the host's launches are
    estimated to take longer than the device's work, and never beyond ``cap``.  (Measured: a 28-layer model of
    0.6 G elements takes 2.04 instead of 2.51 ms for a prompt of 128 tokens; a 36-layer model of 4 G elements is
    bound by the device at 512 tokens, 7.3 ms either way, and gains nothing from the capture.)"""
    if cap <= 0 or matrix_elements <= 0:
        return max(cap, 0)
    host = launches * HOST_SECONDS_PER_LAUNCH
    if matrix_elements * element_bytes / STREAM_BYTES_PER_SECOND >= host:
        return 0
    return int(min(cap, host * PRODUCT_OPS_PER_SECOND / (2.0 * matrix_elements)))


class NotCaptured(RuntimeError):
    """A step ran in its warm-up but its capture as a graph failed."""


@dataclasses.dataclass
class _Captured:
    graph: torch.cuda.CUDAGraph
    buffer: torch.Tensor      # the fixed int32 index buffer
    logits: torch.Tensor      # the graph's output [B, vocab] float32
    stride: int


class StepGraphs:

    SEEN_SHAPES = 512   # shapes of steps with portions remembered as met once

    def __init__(self, engine, max_batch: int, cache_size: int = 32, portion_tokens: int = 0):
        self.engine = weakref.proxy(engine)   # the engine owns this object: no cycle, so both go when the engine is let go
        self.max_batch = int(max_batch)
        self.cache_size = max(1, int(cache_size))
        self.portion_tokens = int(portion_tokens)
        self._graphs: "collections.OrderedDict[tuple, _Captured]" = collections.OrderedDict()
        self._seen: "collections.OrderedDict[tuple, None]" = collections.OrderedDict()
        self._refused: "collections.OrderedDict[tuple, None]" = collections.OrderedDict()   # shapes whose capture failed
        self._pool = None
        self.replays = 0
        self.captures = 0
        self.evictions = 0

    def eligible(self, entries: Sequence, starts: Sequence[int]) -> bool:
        """Whether the step is to be replayed.  A step of single tokens is, from its first time; a step with
        portions from the second time its shape is met (the first time only remembers the shape).  A shape whose
        capture has failed is not tried again."""
        if not 1 <= len(entries) <= self.max_batch:
            return False
        if len(starts) != len(entries):
            raise ValueError(f"{len(entries)} entries but {len(starts)} starts")
        if self._single_tokens(entries):
            return self._key(entries, starts) not in self._refused
        if self.portion_tokens <= 0 or sum(len(e.tokens) for e in entries) > self.portion_tokens:
            return False
        if any(len(e.want) > 1 for e in entries):
            return False       # rows of logits beyond one a request: the graph's own output tensor would be large
        key = self._key(entries, starts)
        if key in self._graphs:
            return True
        if key in self._refused:
            return False
        if key in self._seen:
            del self._seen[key]
            return True
        self._seen[key] = None
        while len(self._seen) > self.SEEN_SHAPES:
            self._seen.popitem(last=False)
        return False

    @staticmethod
    def _single_tokens(entries: Sequence) -> bool:
        return all(len(e.tokens) == 1 and len(e.want) == 1 and int(e.want[0]) == 0 for e in entries)

    def _key(self, entries: Sequence, starts: Sequence[int]) -> tuple:
        counts = tuple(len(e.tokens) for e in entries)
        stride = self._stride_for([s + c for s, c in zip(starts, counts)])
        if self._single_tokens(entries):
            return (len(entries), stride)
        # any other step (portions, or single tokens some of which want no logits): its own kind of key
        portions = [i for i, c in enumerate(counts) if c > 1]
        level = bool(portions) and min(starts[i] for i in portions) >= max(counts)
        return (counts, sum(len(e.want) for e in entries), level, stride)

    def owns(self, t: torch.Tensor) -> bool:
        return any(t is g.logits for g in self._graphs.values())

    def _stride_for(self, ends: Sequence[int]) -> int:
        # the bound the decode kernels round a step's longest context to anyway: a replayed step is then launched
        # exactly as the same step run directly would be
        from ..ops import kernels as K
        page = self.engine.page_size
        return K.decode_context_bound(max(ends), page) // page

    def run(self, entries: Sequence, starts: Sequence[int], carried=None):
        """The step's logits from its graph, captured first if need be.  None if its capture failed (no memory
        for its activations, say): the caller then runs it directly, which gives the same bits, as it will every
        later step of that shape."""
        eng = self.engine
        key = self._key(entries, starts)
        stride = key[-1]
        cap = self._graphs.get(key)
        if cap is None:
            while len(self._graphs) >= self.cache_size:
                # the device may still be replaying it (the host runs a step ahead): wait, then let it go
                torch.cuda.synchronize(eng.device)
                self._graphs.popitem(last=False)
                self.evictions += 1
            try:
                cap = self._capture(entries, starts, stride, carried)
            except NotCaptured:
                self._refused[key] = None
                while len(self._refused) > self.SEEN_SHAPES:
                    self._refused.popitem(last=False)
                return None
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
        size = eng.tables.step_layout(n, sum(len(e.tokens) for e in entries), stride,
                                      sum(len(e.want) for e in entries))["_total"][1]
        buffer = torch.empty(size, dtype=torch.int32, device=eng.device)
        batch = eng.build_batch(entries, starts, stride=stride, device_buffer=buffer, carried=carried)
        # once outside a capture, on a side stream, so that whatever libraries set up lazily exists already;
        # it writes the same keys and values the replay will write.  State of fixed size is not written twice to
        # the same effect (a recurrence would advance two steps): the slots' rows are put back afterwards.
        stateful = [c for c in eng.caches if hasattr(c, "snapshot")] if eng.model.needs_state else []
        saved = [c.snapshot(batch.state_slots) for c in stateful]
        side = torch.cuda.Stream(device=eng.device)
        side.wait_stream(torch.cuda.current_stream())
        try:
            with torch.cuda.stream(side):
                eng.forward(batch)
        finally:
            torch.cuda.current_stream().wait_stream(side)
            for c, rows in zip(stateful, saved):
                c.restore(batch.state_slots, rows)
        torch.cuda.synchronize()
        # The warm-up ran the same launches, so what fails from here on is the capture itself (its pool's memory, an
        # operation that cannot be recorded): the step can still run directly.
        # No cyclic garbage collection while the stream is being captured: a collection runs the destructors of
        # whatever dead cycles the process holds, and the destructor of an earlier engine's graph waits for the
        # device, which is not allowed during a capture and ends the process.  What is dead stays so until after.
        collecting = gc.isenabled()
        gc.disable()
        try:
            graph = torch.cuda.CUDAGraph()
            if self._pool is None:
                self._pool = torch.cuda.graph_pool_handle()
            with torch.cuda.graph(graph, pool=self._pool):
                logits = eng.forward(batch)
        except Exception as e:
            raise NotCaptured(f"a step of {[len(e_.tokens) for e_ in entries]} tokens could not be captured: {e}") from e
        finally:
            if collecting:
                gc.enable()
        self.captures += 1
        return _Captured(graph, buffer, logits, stride)
