"""The cache manager as Python sees it: a thin face over the C++ bookkeeping
(``csrc/host/cache_manager.cpp``) plus the device tensors the pages live in.

Groups: layers whose mixers keep keys and values with the same shape and the
same window share one group: one pool of pages, one block table per request.
A group with a window gives pages back as soon as no later token can see
them.  Beside the pages there is a pool of slots for per-request state of
fixed size (crates/prelude-core/src/scheduler/components/cache/deltanet_pool.rs:54-173),
one slot per live request when the model has a mixer that keeps such state.

What lies in a page is the mixer's business: every cache specification
allocates its own storage (``parts.base.PagedCacheSpec.allocate``; keys and
values: K ``[pages, kv_heads, page_size, head_dim]`` and V transposed, see
``KVCacheSpec``), the manager only counts bytes, hands out pages and builds
the tables.
"""
from __future__ import annotations

import ctypes
import dataclasses
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from .._native import host
from ..parts.base import KVLayerCache, PagedCacheSpec, StateLayerCache   # noqa: F401  (the views are re-exported here)


class CacheError(RuntimeError):
    pass


class OutOfPages(CacheError):
    """A pool has too few free pages for what was asked; nothing was taken."""


def _p(a: np.ndarray):
    return a.ctypes.data_as(ctypes.c_void_p)


class PageTables:
    """Pools, per-request tables and state slots (host side only; no GPU needed)."""

    def __init__(self, page_size: int, groups: Sequence[Tuple[int, int]], state_slots: int = 0):
        """``groups``: (number of pages, window or 0) per group."""
        if page_size < 1:
            raise CacheError(f"page size {page_size} must be positive")
        for n, w in groups:
            if n < 1 or w < 0:
                raise CacheError(f"a cache group needs at least one page and a window >= 0, got ({n}, {w})")
            if n * page_size >= 2 ** 31:
                raise CacheError(f"{n} pages of {page_size} tokens exceed 32-bit slot numbers")
        self._lib = host()
        self.page_size = int(page_size)
        self.groups = [(int(n), int(w)) for n, w in groups]
        n = (ctypes.c_int * len(groups))(*[g[0] for g in self.groups])
        w = (ctypes.c_int * len(groups))(*[g[1] for g in self.groups])
        self._h = self._lib.pa_cache_create(self.page_size, len(self.groups), n, w, int(state_slots))
        if not self._h:
            raise CacheError("cache manager could not be created")

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.pa_cache_destroy(h)

    @property
    def handle(self):
        return self._h

    def _err(self) -> str:
        return self._lib.pa_cache_error(self._h).decode()

    # ---- requests --------------------------------------------------------
    def open(self, rid: int, need_state: bool = False) -> None:
        if self._lib.pa_cache_open(self._h, rid, int(need_state)) != 0:
            raise CacheError(self._err())

    def reserve(self, rid: int, new_len: int) -> None:
        rc = self._lib.pa_cache_reserve(self._h, rid, new_len)
        if rc == 1:
            raise OutOfPages(f"request {rid}: no pages left to reach {new_len} tokens "
                             f"(free per group: {[self.free_pages(g) for g in range(len(self.groups))]})")
        if rc != 0:
            raise CacheError(self._err())

    def commit(self, rid: int, new_len: int) -> None:
        if self._lib.pa_cache_commit(self._h, rid, new_len) != 0:
            raise CacheError(self._err())

    def rollback(self, rid: int) -> None:
        if self._lib.pa_cache_rollback(self._h, rid) != 0:
            raise CacheError(self._err())

    def close(self, rid: int) -> None:
        if self._lib.pa_cache_close(self._h, rid) != 0:
            raise CacheError(self._err())

    def has(self, rid: int) -> bool:
        return bool(self._lib.pa_cache_has(self._h, rid))

    def length(self, rid: int) -> int:
        return self._lib.pa_cache_len(self._h, rid)

    def state_slot(self, rid: int) -> int:
        return self._lib.pa_cache_state_slot(self._h, rid)

    def table(self, rid: int, group: int) -> List[int]:
        n = self._lib.pa_cache_table(self._h, rid, group, None, 0)
        if n < 0:
            raise CacheError(f"request {rid} or group {group} unknown")
        buf = np.empty(max(n, 1), dtype=np.int32)
        self._lib.pa_cache_table(self._h, rid, group, _p(buf), n)
        return buf[:n].tolist()

    # ---- pools -----------------------------------------------------------
    def free_pages(self, group: int) -> int:
        return self._lib.pa_cache_free_pages(self._h, group)

    def capacity_pages(self, group: int) -> int:
        return self._lib.pa_cache_capacity_pages(self._h, group)

    def free_state_slots(self) -> int:
        return self._lib.pa_cache_free_state_slots(self._h)

    def num_requests(self) -> int:
        return self._lib.pa_cache_num_requests(self._h)

    def live_pages(self, rid: int, group: int) -> int:
        return self._lib.pa_cache_live_pages(self._h, rid, group)

    def reservable_len(self, rid: int) -> int:
        return self._lib.pa_cache_reservable_len(self._h, rid)

    def peak_pages(self, total: int, chunk: int, group: int) -> int:
        return self._lib.pa_cache_peak_pages(self._h, total, chunk, group)

    def audit(self) -> str:
        """"" when every page and slot is free or held by exactly one live request, else what is wrong."""
        return self._lib.pa_cache_audit(self._h).decode()

    @staticmethod
    def slot(table: Sequence[int], pos: int, page_size: int) -> int:
        """slot = table[pos / P] * P + pos % P (crates/prelude-core/src/scheduler/components/cache/block_manager.rs:105-109)."""
        return table[pos // page_size] * page_size + pos % page_size

    # ---- one step's index arrays -----------------------------------------
    def step_layout(self, n: int, total: int, stride: int, wanted: int) -> Dict[str, Tuple[int, int]]:
        """Offsets (in int32 elements) of each array inside one packed buffer."""
        G = len(self.groups)
        sizes = [("token_ids", total), ("positions", total), ("seq_of_token", total), ("cu_q", n + 1),
                 ("context_lens", n), ("state_slots", n), ("fresh", n), ("want_rows", wanted),
                 ("decode_seqs", n), ("prefill_seqs", n), ("carry_src", n), ("carry_dst", n),
                 ("block_tables", G * n * stride), ("slots", G * total)]
        out, off = {}, 0
        for name, sz in sizes:
            out[name] = (off, sz)
            off += sz
        out["_total"] = (0, off)
        return out

    def fill_step(self, ids: Sequence[int], starts: Sequence[int], counts: Sequence[int], stride: int,
                  buf: np.ndarray, layout: Dict[str, Tuple[int, int]]) -> None:
        n = len(ids)
        a_ids = np.asarray(ids, dtype=np.int64)
        a_st = np.asarray(starts, dtype=np.int32)
        a_ct = np.asarray(counts, dtype=np.int32)

        def at(name):
            off, _ = layout[name]
            return ctypes.c_void_p(buf.ctypes.data + 4 * off)

        rc = self._lib.pa_cache_fill_step(self._h, n, _p(a_ids), _p(a_st), _p(a_ct), stride, at("positions"),
                                          at("seq_of_token"), at("cu_q"), at("context_lens"), at("state_slots"),
                                          at("fresh"), at("block_tables"), at("slots"))
        if rc != 0:
            raise CacheError(self._err())


def _paged(cs) -> bool:
    return bool(getattr(cs, "PAGED", False))


def plan_groups(cache_specs: Sequence[object]) -> Tuple[List[PagedCacheSpec], List[Optional[int]]]:
    """Groups the model's cache slots: paged specs that compare equal share a group (``PagedCacheSpec``).
    Returns the groups' specs and, per cache slot, its group (None for slots of per-request state)."""
    groups: List[PagedCacheSpec] = []
    of_slot: List[Optional[int]] = []
    for cs in cache_specs:
        if _paged(cs):
            if cs not in groups:
                groups.append(cs)
            of_slot.append(groups.index(cs))
        else:
            of_slot.append(None)
    return groups, of_slot


def bytes_per_token(cache_specs: Sequence[object], dtype: torch.dtype) -> int:
    el = torch.empty((), dtype=dtype).element_size()
    return sum(int(cs.bytes_per_token(el)) for cs in cache_specs if _paged(cs))


def state_bytes_per_slot(cache_specs: Sequence[object]) -> int:
    """Bytes one request's state of fixed size takes, over all cache slots that keep such state."""
    return sum(int(cs.bytes_per_slot()) for cs in cache_specs if not _paged(cs))


def peak_pages(total: int, chunk: int, window: int, page_size: int) -> int:
    """Pages of a group with this window that a request of ``total`` tokens holds at most when it is fed in
    portions of at most ``chunk`` tokens (the rule of ``CacheManager::peak_pages``)."""
    pages = lambda n: -(-n // page_size)
    if window <= 0:
        return pages(total)
    return min(pages(total), pages(max(1, chunk) + window - 1) + 1)


def pages_per_group(tokens: int, group_specs: Sequence[PagedCacheSpec], page_size: int, max_requests: int,
                    max_request_tokens: int, chunk: int) -> List[int]:
    """Pages each group needs so that live requests can hold ``tokens`` tokens between them: a group that
    sees every key holds them all; one with a window holds per request what the window and a portion span,
    so it needs no more than that for as many requests as may run."""
    full = max(1, -(-tokens // page_size))
    out = []
    for g in group_specs:
        if g.window > 0:
            out.append(max(1, min(full, max_requests * peak_pages(max_request_tokens, chunk, g.window, page_size))))
        else:
            out.append(full)
    return out


def allocate_storage(cache_specs: Sequence[object], of_slot: Sequence[Optional[int]], pages_per_group: Sequence[int],
                     page_size: int, state_slots: int, dtype: torch.dtype, device: torch.device) -> List[object]:
    """Device storage for every cache slot, zero-initialised: each specification allocates its own kind
    (``PagedCacheSpec.allocate`` / ``SlotCacheSpec.allocate``)."""
    out: List[object] = []
    for cs, g in zip(cache_specs, of_slot):
        if not callable(getattr(cs, "allocate", None)):
            raise CacheError(f"unknown cache specification {cs!r}: it has no allocate()")
        if _paged(cs):
            out.append(cs.allocate(pages_per_group[g], page_size, dtype, device, g))
        else:
            out.append(cs.allocate(state_slots, device))
    return out
