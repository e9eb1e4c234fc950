"""A decoder assembled from a ``ModelSpec``: embedding, the layers in their run
order, final norm on the wanted rows, output head.

Counterpart of the reference's hand-written model
(crates/prelude-core/src/models/qwen3.rs:534-660: embed, layers carrying
(hidden, residual), final norm of hidden + residual, last-token select, head),
except that the structure is read from data and the head runs only on the rows
whose logits are wanted.
"""
from __future__ import annotations

import dataclasses
from typing import Dict, List, Optional, Tuple

import torch

from ..parts import Block, Part, TensorReq, build_part
from ..parts.base import PartError, _REGISTRY
from .spec import ModelSpec, PartSpec


@dataclasses.dataclass
class CacheSlot:
    """What one run of a layer keeps between steps."""
    run: int                    # index in the run order that owns (writes) it
    spec: object                # a PagedCacheSpec (keys and values, or a kind of the mixer's own) | a SlotCacheSpec


class CausalLM:
    def __init__(self, spec: ModelSpec):
        spec.validate()
        self.spec = spec
        self.dtype: Optional[torch.dtype] = None
        self.device: Optional[torch.device] = None
        # (part, its spec) in a fixed order, for tensor requests and loading
        self._parts: List[Tuple[Part, PartSpec]] = []
        self.shared: Dict[str, Part] = {}
        for name, ps in spec.positions.items():
            p = build_part("position", ps.kind, ps.params)
            self.shared[name] = p
            self._parts.append((p, ps))
        self.embedding = self._make("embedding", spec.embedding)
        self.blocks: List[Block] = []
        for ls in spec.layers:
            cls = _REGISTRY.get(("block", ls.block))
            if cls is None:
                raise PartError(f"no block of kind {ls.block!r} is registered")
            subs = {}
            for slot, category in cls.SLOTS.items():
                if slot not in ls.parts:
                    raise PartError(f"block {ls.block!r} needs a part for its slot {slot!r}")
                subs[slot] = self._make(category, ls.parts[slot])
            extra = set(ls.parts) - set(cls.SLOTS)
            if extra:
                raise PartError(f"block {ls.block!r} has no slots {sorted(extra)}")
            self.blocks.append(build_part("block", ls.block, ls.block_params, **subs))
        self.final_norm = self._make("norm", spec.final_norm)
        self.head = self._make("head", spec.head)
        for p, _ in self._parts:
            p.bind(self.shared)

        # caches: one per run that does not read another's
        self.cache_slots: List[Optional[CacheSlot]] = []
        self.run_cache: List[Optional[int]] = []   # run index -> index into cache_slots
        for i, r in enumerate(spec.order):
            mixer = getattr(self.blocks[r.layer], "mixer", None)
            cs = mixer.cache_spec() if mixer is not None else None
            if r.reads_cache_of is not None:
                src = self.run_cache[r.reads_cache_of]
                if src is None or self.cache_slots[src].spec != cs:
                    raise PartError(f"run {i} cannot read the cache of run {r.reads_cache_of}: "
                                    f"it keeps {self.cache_slots[src].spec if src is not None else None}, "
                                    f"this layer needs {cs}")
                self.run_cache.append(src)
            elif cs is None:
                self.run_cache.append(None)
            else:
                self.cache_slots.append(CacheSlot(i, cs))
                self.run_cache.append(len(self.cache_slots) - 1)

    def _make(self, category: str, ps: PartSpec) -> Part:
        p = build_part(category, ps.kind, ps.params)
        self._parts.append((p, ps))
        return p

    # ---- tensors ---------------------------------------------------------
    def tensor_requests(self) -> Dict[str, TensorReq]:
        """Checkpoint tensor name -> what is required of it, over all parts."""
        out: Dict[str, TensorReq] = {}
        for part, ps in self._parts:
            for local, req in part.tensors().items():
                if local not in ps.weights:
                    raise PartError(f"{ps.kind}: no checkpoint name given for its tensor {local!r}")
                name = ps.weights[local]
                if name in out and out[name] != req:
                    raise PartError(f"tensor {name!r} is asked for as {out[name]} and as {req}")
                out[name] = req
        return out

    def load(self, fetch, dtype: torch.dtype, device: torch.device) -> None:
        """``fetch(checkpoint_name, req)`` returns the tensor on the device in the type its kind asks for."""
        self.dtype, self.device = dtype, device
        for part, ps in self._parts:
            tensors = {local: fetch(ps.weights[local], req) for local, req in part.tensors().items()}
            part.load(tensors, dtype, device)
        for p in self.shared.values():
            p.prepare(device)

    def matrix_elements(self) -> int:
        """Elements of the weight matrices a step multiplies with (the embedding table is only looked up in)."""
        from ..parts.base import MATRIX
        seen, total = set(), 0
        for part, ps in self._parts:
            if part is self.embedding:
                continue
            for local, req in part.tensors().items():
                if req.kind == MATRIX and ps.weights[local] not in seen:
                    seen.add(ps.weights[local])
                    n = 1
                    for d in req.shape:
                        n *= int(d)
                    total += n
        return total

    def launches_per_step(self) -> int:
        """Kernel launches of one step, about: every run's block by its parts' own counts, and the embedding, the
        final norm and the head."""
        total = self.embedding.LAUNCHES + self.final_norm.LAUNCHES + self.head.LAUNCHES
        for r in self.spec.order:
            b = self.blocks[r.layer]
            total += b.launches() if hasattr(b, "launches") else 1
        return total

    # ---- what the cache manager must provide ------------------------------
    @property
    def needs_state(self) -> bool:
        return any(not getattr(c.spec, "PAGED", False) for c in self.cache_slots)

    @property
    def graph_safe(self) -> bool:
        """Whether a decode step may be captured once and replayed: no part says no."""
        return all(p.GRAPH_SAFE for p, _ in self._parts) and all(b.GRAPH_SAFE for b in self.blocks)

    @property
    def graph_safe_portions(self) -> bool:
        """Whether a step that brings prompt portions may be captured and replayed too: every part says yes."""
        return self.graph_safe and all(p.GRAPH_SAFE_PORTIONS for p, _ in self._parts) and \
            all(b.GRAPH_SAFE_PORTIONS for b in self.blocks)

    @property
    def atomic_prefill(self) -> bool:
        """Whether some mixer cannot continue a prompt from a cut: requests are then fed whole or not at all."""
        return any(getattr(p, "ATOMIC_PREFILL", False) for p, _ in self._parts)

    # ---- forward ------------------------------------------------------------
    def forward(self, step, caches) -> torch.Tensor:
        """Runs the step's tokens; returns float32 logits [W, vocab] at ``step.want_rows``.

        ``caches[i]`` is the view of cache slot i (``engine.caches``).
        """
        hidden = self.embedding.forward(step.token_ids)
        residual = None
        for i, r in enumerate(self.spec.order):
            ci = self.run_cache[i]
            cache = caches[ci] if ci is not None else None
            hidden, residual = self.blocks[r.layer].forward(hidden, residual, step, cache,
                                                            write_cache=r.reads_cache_of is None)
        if step.want_rows.shape[0] == 0:
            return torch.empty((0, self.spec.vocab_size), dtype=torch.float32, device=hidden.device)
        if not self.final_norm.TAKES_SLICE_SUMS:
            from ..ops import kernels as K
            hidden = K.as_tensor(hidden)
        normed = self.final_norm.forward_rows(hidden, residual, step.want_rows)
        return self.head.forward(normed)
