"""The scheduler as Python sees it: a face over ``csrc/host/scheduler.cpp``.

It admits requests, cuts what each still has to feed into portions under one
token budget per step, and decides what happens when pages run out; see the
C++ header for the policy and the reference lines it follows.
"""
from __future__ import annotations

import ctypes
import dataclasses
from typing import List

import numpy as np

from .._native import host
from ..cache.manager import PageTables


class SchedulerError(RuntimeError):
    pass


@dataclasses.dataclass
class Portion:
    id: int
    start: int      # first position fed
    count: int      # tokens fed
    samples: bool   # the last fed token is the last one known: a new token is drawn from its logits


@dataclasses.dataclass
class SequenceInfo:
    known: int
    computed: int
    generated: int
    max_new: int
    preempt_count: int
    running: bool


class Scheduler:
    def __init__(self, tables: PageTables, max_num_batched_tokens: int = 8192, long_prefill_token_threshold: int = 0,
                 max_running_requests: int = 256, max_total_tokens: int = 0, decode_reservation_cap: int = 4096,
                 decode_priority_max_remaining_tokens: int = 4, needs_state: bool = False):
        self._lib = host()
        self._tables = tables   # keeps the cache manager alive as long as the scheduler
        self._h = self._lib.pa_sched_create(tables.handle, max_num_batched_tokens, long_prefill_token_threshold,
                                            max_running_requests, max_total_tokens, decode_reservation_cap,
                                            decode_priority_max_remaining_tokens, int(needs_state))
        self._cap = 0
        self._grow(1024)

    def _grow(self, cap: int) -> None:
        self._cap = cap
        self._ids = np.empty(cap, dtype=np.int64)
        self._starts = np.empty(cap, dtype=np.int32)
        self._counts = np.empty(cap, dtype=np.int32)
        self._samples = np.empty(cap, dtype=np.int32)

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.pa_sched_destroy(h)

    def _err(self) -> str:
        return self._lib.pa_sched_error(self._h).decode()

    def add_request(self, rid: int, prompt_len: int, max_new: int, atomic: bool = False, max_chunk: int = 0) -> None:
        """``atomic``: what the request has to feed is fed whole in one step or not at all (for mixers that
        cannot continue a prompt from a cut); ``max_chunk``: a cap on its portions, 0 = none."""
        if self._lib.pa_sched_add(self._h, rid, prompt_len, max_new, int(bool(atomic)), int(max_chunk)) != 0:
            raise SchedulerError(self._err())

    def schedule(self) -> List[Portion]:
        """Decides the next step and reserves its pages; [] when nothing can run."""
        need = self.num_running + self.num_waiting + 1
        if need > self._cap:
            self._grow(2 * need)
        p = lambda a: a.ctypes.data_as(ctypes.c_void_p)
        n = self._lib.pa_sched_schedule(self._h, p(self._ids), p(self._starts), p(self._counts), p(self._samples),
                                        self._cap)
        if n < 0:
            raise SchedulerError("schedule: more entries than requests")
        err = self._err()
        if n == 0 and err:
            raise SchedulerError(err)
        return [Portion(int(self._ids[i]), int(self._starts[i]), int(self._counts[i]), bool(self._samples[i]))
                for i in range(n)]

    def step_done(self) -> None:
        if self._lib.pa_sched_step_done(self._h) != 0:
            raise SchedulerError(self._err())

    def step_cancelled(self) -> None:
        self._lib.pa_sched_step_cancelled(self._h)

    def on_token(self, rid: int) -> None:
        if self._lib.pa_sched_on_token(self._h, rid) != 0:
            raise SchedulerError(self._err())

    def finish(self, rid: int) -> None:
        if self._lib.pa_sched_finish(self._h, rid) != 0:
            raise SchedulerError(self._err())

    @property
    def num_waiting(self) -> int:
        return self._lib.pa_sched_num_waiting(self._h)

    @property
    def num_running(self) -> int:
        return self._lib.pa_sched_num_running(self._h)

    @property
    def tokens_in_use(self) -> int:
        return self._lib.pa_sched_tokens_in_use(self._h)

    @property
    def preemptions(self) -> int:
        return self._lib.pa_sched_preemptions(self._h)

    def last_preempted(self) -> List[int]:
        buf = np.empty(max(1, self.num_waiting + self.num_running), dtype=np.int64)
        n = self._lib.pa_sched_last_preempted(self._h, buf.ctypes.data_as(ctypes.c_void_p), len(buf))
        return buf[:min(n, len(buf))].tolist()

    def info(self, rid: int) -> SequenceInfo:
        out = (ctypes.c_int * 6)()
        if self._lib.pa_sched_info(self._h, rid, out) != 0:
            raise SchedulerError(f"request {rid} is unknown")
        return SequenceInfo(out[0], out[1], out[2], out[3], out[4], bool(out[5]))

    def has_work(self) -> bool:
        return self.num_running + self.num_waiting > 0
