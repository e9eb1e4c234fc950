"""The model with its cache on one GPU, and the one step function everything drives.

``Engine.step`` takes a batch of (request, its next tokens, the places whose
logits are wanted): portions of prompts beside single decoded tokens, cut
anywhere.  It runs exactly the tokens it is given, as one packed batch, from
the cache earlier steps left, and returns the logits at the wanted places.
The reference's counterpart is ``batch_mixed_paged``
(crates/prelude-core/src/engine/model_runner/paged_mixed.rs:13-335) over
``StepRequest`` (crates/prelude-core/src/engine/executor.rs:96-115), which
always returns one row per request.
"""
from __future__ import annotations

import dataclasses
from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import (CacheError, PageTables, allocate_storage, bytes_per_token, pages_per_group,
                             plan_groups, state_bytes_per_slot)
from ..config.engine_config import EngineConfig
from ..config.model_config import read_config_json
from ..config.registry import resolve_architecture
from ..models.causal_lm import CausalLM
from ..weights.loader import load_into
from .batch import GroupStep, StepBatch


class StepError(ValueError):
    pass


@dataclasses.dataclass
class StepEntry:
    """One request's share of a step."""
    id: int
    tokens: Sequence[int]
    want: Sequence[int] = ()     # indices into ``tokens`` whose logits are wanted
    carry: Optional[int] = None  # the last of ``tokens`` is a stand-in: its id is row ``carry`` of the step's ``carried``


class _Staging:
    """Pinned host buffers for the step's index arrays, used in turn so that a
    buffer is rewritten only after the copy that read it has finished."""

    def __init__(self, depth: int = 3):
        self._bufs: List[Optional[torch.Tensor]] = [None] * depth
        self._events: List[Optional[torch.cuda.Event]] = [None] * depth
        self._i = 0

    def get(self, n: int) -> tuple:
        i = self._i
        self._i = (i + 1) % len(self._bufs)
        if self._events[i] is not None:
            self._events[i].synchronize()
        b = self._bufs[i]
        if b is None or b.numel() < n:
            b = torch.empty(max(4096, 2 * n), dtype=torch.int32, pin_memory=True)
            self._bufs[i] = b
        return i, b

    def sent(self, i: int) -> None:
        ev = torch.cuda.Event()
        ev.record()
        self._events[i] = ev


class Engine:
    def __init__(self, model: CausalLM, config: EngineConfig, raw_config: Optional[dict] = None):
        """``model`` must be loaded (``weights.load_into``) on ``config.device``."""
        if model.device is None:
            raise StepError("the model has no weights loaded")
        self.model = model
        self.config = config
        self.raw_config = raw_config or {}
        self.device = model.device
        self.dtype = model.dtype
        self.vocab_size = model.spec.vocab_size
        self.max_positions = model.spec.max_positions
        self.page_size = int(config.page_size)
        specs = [c.spec for c in model.cache_slots]
        self.group_specs, self._group_of_slot = plan_groups(specs)
        self._staging = _Staging()
        self._live: Dict[int, int] = {}   # request id -> tokens fed so far
        self._graphs = None
        state_slots = config.max_state_slots if model.needs_state else 0
        self.memory_plan: Dict[str, int] = {}
        tokens = self._decide_cache_tokens(specs, state_slots)
        pages = self._pages_for(tokens)
        self.cache_tokens = max(pages) * self.page_size if pages else self.page_size
        self._set_cache(pages, state_slots)
        # decode steps as HIP graphs, in the serving type, for models none of whose parts says it cannot be replayed
        if config.hip_graph and model.graph_safe and self.dtype == torch.bfloat16:
            from .graph import StepGraphs
            self._graphs = StepGraphs(self, config.hip_graph_max_bs, config.hip_graph_cache_size,
                                        self._graph_portion_tokens())

    def _chunk_cap(self) -> int:
        """The most tokens of one request a step may bring."""
        cap = int(self.config.max_num_batched_tokens)
        if self.config.long_prefill_token_threshold > 0:
            cap = min(cap, int(self.config.long_prefill_token_threshold))
        return max(1, cap)

    def _pages_for(self, tokens: int) -> List[int]:
        return pages_per_group(tokens, self.group_specs, self.page_size, max(1, int(self.config.max_running_requests)),
                               self.max_positions, self._chunk_cap())

    def _set_cache(self, pages: List[int], state_slots: int) -> None:
        specs = [c.spec for c in self.model.cache_slots]
        self.tables = PageTables(self.page_size, [(n, g.window) for n, g in zip(pages, self.group_specs)], state_slots)
        self.caches = allocate_storage(specs, self._group_of_slot, pages, self.page_size, state_slots, self.dtype,
                                       self.device)
        self.pages_per_group = list(pages)

    # ---- construction -------------------------------------------------------
    @classmethod
    def from_model_dir(cls, model_dir: str, config: Optional[EngineConfig] = None) -> "Engine":
        """Reads config.json, picks the architecture from the registry, loads the safetensors."""
        from .. import models  # noqa: F401  registers the built-in architectures
        config = config or EngineConfig()
        if not torch.cuda.is_available():
            raise RuntimeError("prelude_amd needs a GPU: torch sees no HIP device, and there is no CPU path")
        raw = read_config_json(model_dir)
        arch = resolve_architecture(raw)
        model = CausalLM(arch.build_spec(arch.parse_config(raw)))
        device = torch.device(config.device)
        torch.cuda.set_device(device)
        from ..ops import kernels as K
        K.set_weight_tiles(config.weight_tiles)
        load_into(model, model_dir, config.torch_dtype(), device)
        return cls(model, config, raw)

    @classmethod
    def from_config(cls, raw_config: dict, config: Optional[EngineConfig] = None, seed: int = 0, std: float = 0.02,
                    norm_std: float = 0.01) -> "Engine":
        """The random-weights mode without a folder: the architecture ``raw_config`` (a config.json's content)
        names, with every tensor drawn on the device from (seed, tensor name)."""
        from .. import models  # noqa: F401
        from ..weights.random_init import load_random
        config = config or EngineConfig()
        if not torch.cuda.is_available():
            raise RuntimeError("prelude_amd needs a GPU: torch sees no HIP device, and there is no CPU path")
        arch = resolve_architecture(raw_config)
        model = CausalLM(arch.build_spec(arch.parse_config(raw_config)))
        device = torch.device(config.device)
        torch.cuda.set_device(device)
        from ..ops import kernels as K
        K.set_weight_tiles(config.weight_tiles)
        load_random(model, config.torch_dtype(), device, seed, std, norm_std)
        return cls(model, config, dict(raw_config))

    def _graph_portion_tokens(self) -> int:
        """Up to how many tokens a step with portions is replayed from a graph (0: such steps never are)."""
        from .graph import portion_tokens_worth_a_graph
        if not (self.config.hip_graph and self.model.graph_safe_portions and self.dtype == torch.bfloat16):
            return 0
        return portion_tokens_worth_a_graph(self.model.matrix_elements(), self.model.launches_per_step(), 2,
                                            int(self.config.hip_graph_portion_tokens))

    def _cache_bytes(self, tokens: int, specs) -> int:
        """Bytes the pages take when live requests may hold ``tokens`` tokens (windowed groups are bounded)."""
        el = torch.empty((), dtype=self.dtype).element_size()
        pages = self._pages_for(tokens)
        total = 0
        for cs, g in zip(specs, self._group_of_slot):
            if g is not None:
                total += pages[g] * self.page_size * int(cs.bytes_per_token(el))
        return total

    def _decide_cache_tokens(self, specs, state_slots: int) -> int:
        """How many tokens the page pools hold.  Given (``max_cache_tokens``), or what the device has left after
        the weights, one step's activations as measured by running one, and stated reserves -- the reference's
        rule, crates/prelude-core/src/scheduler/components/cache/manager.rs:240-280 with the dummy forward of
        crates/prelude-core/src/engine/loading.rs:283-368:

            pages = total * gpu_memory_utilization - in use (weights) - peak of a step - reserves

        The reserves are what is allocated only later: the library product's workspace, the state slots, and for
        captured decode steps a logits tensor per kept graph plus their shared activation pool."""
        if self.config.max_cache_tokens is not None:
            return max(int(self.config.max_cache_tokens), self.page_size)
        per_token = bytes_per_token(specs, self.dtype)
        if per_token == 0:
            return self.page_size
        from ..ops import kernels as K
        peak = self._probe_step_bytes(specs, state_slots)
        torch.cuda.synchronize(self.device)
        torch.cuda.empty_cache()
        free, total = torch.cuda.mem_get_info(self.device)
        in_use = total - free
        reserve_state = state_slots * state_bytes_per_slot(specs)
        reserve_library = 0 if self.dtype != torch.bfloat16 else K.library_workspace_reserve(self.device)
        reserve_graphs = 0
        if self.config.hip_graph and self.model.graph_safe and self.dtype == torch.bfloat16:
            logits = int(self.config.hip_graph_max_bs) * self.vocab_size * 4
            reserve_graphs = int(self.config.hip_graph_cache_size) * logits + (256 << 20)
            # captured steps with portions keep their activations in the graphs' shared pool: what the measured
            # step took, in proportion to the tokens such a step may have
            probed = max(1, min(self._chunk_cap(), self.max_positions))
            reserve_graphs += peak * min(probed, self._graph_portion_tokens()) // probed
        budget = int(total * self.config.gpu_memory_utilization) - in_use - peak - reserve_state - reserve_library \
            - reserve_graphs
        self.memory_plan = dict(total=total, in_use=in_use, step_peak=peak, state=reserve_state,
                                library_workspace=reserve_library, graphs=reserve_graphs, cache=max(budget, 0))
        ceiling = self.max_positions * max(1, int(self.config.max_running_requests))
        floor = 16 * self.page_size
        if budget <= self._cache_bytes(floor, specs):
            return floor
        lo, hi = floor, ceiling          # the most tokens whose pages fit the budget (the cost grows with the tokens)
        if self._cache_bytes(hi, specs) <= budget:
            return hi
        while hi - lo > self.page_size:
            mid = (lo + hi) // 2
            if self._cache_bytes(mid, specs) <= budget:
                lo = mid
            else:
                hi = mid
        return lo // self.page_size * self.page_size

    def _probe_step_bytes(self, specs, state_slots: int) -> int:
        """Runs one step of as many tokens as a step may bring (one request, its last rows wanted) over a cache
        just large enough for it, and returns the peak of device memory the step took beyond what was
        allocated before it; the cache is given back."""
        n = max(1, min(self._chunk_cap(), self.max_positions))
        rows = min(n, max(512, int(self.config.max_running_requests)))
        pages = [max(1, -(-n // self.page_size))] * len(self.group_specs)
        self._set_cache(pages, 1 if state_slots else 0)
        torch.cuda.synchronize(self.device)
        before = torch.cuda.memory_allocated(self.device)
        torch.cuda.reset_peak_memory_stats(self.device)
        try:
            self.step([StepEntry(-1, [0] * n, list(range(n - rows, n)))])
            torch.cuda.synchronize(self.device)
            peak = torch.cuda.max_memory_allocated(self.device) - before
        finally:
            self.release(-1)
            self.tables = None
            self.caches = None
        return max(int(peak), 0)

    # ---- requests ---------------------------------------------------------------
    def has(self, rid: int) -> bool:
        return self.tables.has(rid)

    def length(self, rid: int) -> int:
        return self.tables.length(rid)

    def release(self, rid: int) -> None:
        """The request is over: its pages and its state slot go back."""
        if self.tables.has(rid):
            self.tables.close(rid)
        self._live.pop(rid, None)

    # ---- the step -----------------------------------------------------------------
    def step(self, entries: Sequence[StepEntry], carried: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Opens unknown requests, takes pages, runs, and records the new lengths.

        Returns float32 logits [sum(len(want)), vocab] in the order of the
        entries and of each entry's ``want``.  Raises ``OutOfPages`` (with
        nothing taken and nothing run) if the pools cannot hold the step.

        ``carried`` is an int32 device tensor of token ids the host has not
        read yet (the previous step's samples): an entry with ``carry`` set
        takes its last token from there, on the device, so this step can be
        launched while the previous one still runs.
        """
        self._validate(entries, carried)
        opened, reserved = [], []
        try:
            for e in entries:
                if not self.tables.has(e.id):
                    self.tables.open(e.id, self.model.needs_state)
                    opened.append(e.id)
                self.tables.reserve(e.id, self.tables.length(e.id) + len(e.tokens))
                reserved.append(e.id)
        except CacheError:
            for rid in reserved:
                self.tables.rollback(rid)
            for rid in opened:
                self.tables.close(rid)
            raise
        starts = [self.tables.length(e.id) for e in entries]
        try:
            logits = self.run(entries, starts, carried)
        except Exception:
            for e in entries:
                self.tables.rollback(e.id)
            for rid in opened:
                self.tables.close(rid)
            raise
        for e, s in zip(entries, starts):
            self.tables.commit(e.id, s + len(e.tokens))
        if self._graphs is not None and self._graphs.owns(logits):
            logits = logits.clone()   # the graph's own output tensor is overwritten by the next replay
        return logits

    def _validate(self, entries: Sequence[StepEntry], carried: Optional[torch.Tensor] = None) -> None:
        if not entries:
            raise StepError("a step needs at least one entry")
        self._validate_carried(entries, carried)
        total = sum(len(e.tokens) for e in entries)
        if total > self.config.max_num_batched_tokens:
            raise StepError(f"the step brings {total} tokens; max_num_batched_tokens is "
                            f"{self.config.max_num_batched_tokens} (pools and activation memory are sized for that)")
        seen = set()
        for e in entries:
            if e.id in seen:
                raise StepError(f"request {e.id} appears twice in one step")
            seen.add(e.id)
            n = len(e.tokens)
            if n == 0:
                raise StepError(f"request {e.id} brings no tokens")
            a = np.asarray(e.tokens, dtype=np.int64)
            if a.ndim != 1 or int(a.min()) < 0 or int(a.max()) >= self.vocab_size:
                bad = [int(t) for t in a.reshape(-1) if not 0 <= int(t) < self.vocab_size][:1]
                raise StepError(f"request {e.id}: token id {bad[0] if bad else a} is outside the vocabulary "
                                f"of {self.vocab_size}")
            for w in e.want:
                if not 0 <= int(w) < n:
                    raise StepError(f"request {e.id}: wanted place {w} is outside its {n} tokens")
            have = self.tables.length(e.id) if self.tables.has(e.id) else 0
            if have + n > self.max_positions:
                raise StepError(f"request {e.id}: {have} + {n} tokens exceed max_position_embeddings "
                                f"{self.max_positions}")

    def _validate_carried(self, entries: Sequence[StepEntry], carried: Optional[torch.Tensor]) -> None:
        rows = [e.carry for e in entries if e.carry is not None]
        if not rows:
            return
        if carried is None:
            raise StepError("an entry carries a token from the device but the step was given no carried tensor")
        if carried.dtype != torch.int32 or carried.dim() != 1 or carried.device != self.device:
            raise StepError(f"carried token ids must be a 1-d int32 tensor on {self.device}")
        for r in rows:
            if not 0 <= int(r) < carried.shape[0]:
                raise StepError(f"carried row {r} is outside the {carried.shape[0]} token ids carried")

    def build_batch(self, entries: Sequence[StepEntry], starts: Sequence[int], stride: Optional[int] = None,
                    device_buffer: Optional[torch.Tensor] = None,
                    carried: Optional[torch.Tensor] = None) -> StepBatch:
        """Index arrays of the step, built on the host in one pinned buffer and sent in one copy.

        ``stride`` widens the block tables beyond what the step needs and
        ``device_buffer`` receives the arrays instead of a fresh tensor: a
        captured graph reads its inputs from fixed addresses with a fixed layout.
        """
        n = len(entries)
        counts = [len(e.tokens) for e in entries]
        total = sum(counts)
        ends = [s + c for s, c in zip(starts, counts)]
        need = max(1, -(-max(ends) // self.page_size))
        stride = need if stride is None else stride
        if stride < need:
            raise StepError(f"block table stride {stride} is smaller than the {need} pages the step needs")
        wanted = sum(len(e.want) for e in entries)
        layout = self.tables.step_layout(n, total, stride, wanted)
        size = layout["_total"][1]
        slot, pinned = self._staging.get(size)
        host = pinned.numpy()
        off, _ = layout["token_ids"]
        woff, _ = layout["want_rows"]
        csoff, _ = layout["carry_src"]
        cdoff, _ = layout["carry_dst"]
        t = 0
        w = 0
        carries = 0
        for i, (e, c) in enumerate(zip(entries, counts)):
            host[off + t: off + t + c] = e.tokens
            for x in e.want:
                host[woff + w] = t + int(x)
                w += 1
            t += c
            if e.carry is None:
                host[csoff + i] = -1
                host[cdoff + i] = -1
            else:
                host[csoff + i] = int(e.carry)
                host[cdoff + i] = t - 1
                carries += 1
        self.tables.fill_step([e.id for e in entries], starts, counts, stride, host, layout)
        dec = [i for i, c in enumerate(counts) if c == 1]
        pre = [i for i, c in enumerate(counts) if c > 1]
        doff, _ = layout["decode_seqs"]
        poff, _ = layout["prefill_seqs"]
        host[doff: doff + len(dec)] = dec
        host[poff: poff + len(pre)] = pre
        soff, _ = layout["state_slots"]
        foff, _ = layout["fresh"]
        state_host = host[soff: soff + n].tolist()
        fresh_host = host[foff: foff + n].tolist()
        if device_buffer is None:
            dev = torch.empty(size, dtype=torch.int32, device=self.device)
        else:
            if device_buffer.numel() != size:
                raise StepError(f"the fixed index buffer holds {device_buffer.numel()} words, the step needs {size}")
            dev = device_buffer
        dev.copy_(pinned[:size], non_blocking=True)
        self._staging.sent(slot)

        def view(name):
            o, s = layout[name]
            return dev[o: o + s]

        if carries:
            from ..ops import kernels as K
            self._validate_carried(entries, carried)
            K.carry_tokens(carried, view("carry_src"), view("carry_dst"), view("token_ids"))
        max_pre = max([counts[i] for i in pre], default=0)
        min_pre = min([starts[i] for i in pre], default=0)
        level = bool(pre) and min_pre >= max_pre
        replayable = bool(dec) and self._graphs is not None and total <= self._graphs.portion_tokens
        G = len(self.group_specs)
        bt = view("block_tables").view(G, n, stride) if G else None
        sl = view("slots").view(G, total) if G else None
        kv = [GroupStep(bt[g], sl[g]) for g in range(G)]
        fixed = device_buffer is not None
        return StepBatch(num_tokens=total, num_seqs=n, token_ids=view("token_ids"), positions=view("positions"),
                         seq_of_token=view("seq_of_token"), cu_q=view("cu_q"), context_lens=view("context_lens"),
                         state_slots=view("state_slots"), fresh=view("fresh"), want_rows=view("want_rows"), kv=kv,
                         q_lens=counts, starts=list(starts), state_slots_host=state_host, fresh_host=fresh_host,
                         max_q_len=max(counts), max_context_len=stride * self.page_size if fixed else max(ends),
                         page_size=self.page_size,
                         decode_seqs=view("decode_seqs")[:len(dec)], prefill_seqs=view("prefill_seqs")[:len(pre)],
                         n_decode=len(dec), n_prefill=len(pre), max_prefill_q=max_pre,
                         # with fixed buffers the launch shapes must not follow the data.  The fewest tokens behind
                         # a portion only says whether every portion has its own length behind it; the decode
                         # kernels are bound by what the tables can hold.  A step small enough to be replayed one
                         # day is bound the same way when it runs directly (by its longest sequence of either
                         # kind, which rounds to the table's width), so that both give the same bits; a larger
                         # step by its decoding sequences alone, which keeps its workspace small.
                         min_prefill_prefix=((max_pre if level else 0) if fixed else min_pre),
                         max_decode_context=(stride * self.page_size if fixed else
                                             (max(ends) if replayable else max([ends[i] for i in dec], default=0))))

    def run(self, entries: Sequence[StepEntry], starts: Sequence[int],
            carried: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Runs a step whose pages are already reserved (the scheduler's path).

        A step of single tokens whose logits are all wanted is replayed from a
        captured HIP graph when graphs are on, and so is a small step with
        prompt portions whose shape has been met before; the logits tensor it
        returns is then the graph's own and is overwritten by the next such step.
        """
        if self._graphs is not None and self._graphs.eligible(entries, starts):
            logits = self._graphs.run(entries, starts, carried)
            if logits is not None:
                return logits
        batch = self.build_batch(entries, starts, carried=carried)
        return self.forward(batch, any(batch.fresh_host))

    def forward(self, batch: StepBatch, maybe_fresh: bool = True) -> torch.Tensor:
        """The model over a built batch.  State of fixed size starts from zero for the sequences that start their
        request, decided on the device from the step's own arrays (``maybe_fresh`` false spares the launches
        when the host knows that none does; a captured step always carries them)."""
        if self.model.needs_state and maybe_fresh:
            for c in self.caches:
                if hasattr(c, "zero_fresh"):
                    c.zero_fresh(batch.state_slots, batch.fresh)
        return self.model.forward(batch, self.caches)
