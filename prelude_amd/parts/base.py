"""What every part of a layer is, and the registry parts are built from.

A model is described as data (``prelude_amd.models.spec``): each layer names
its parts by *kind* with their sizes and constants as parameters.  A part
knows nothing of the model it sits in: it gets its parameters, says which
tensors it needs (by local name and shape), receives them, and runs.

Categories and the interface each must have:

``norm``      ``forward(x)``, ``forward_residual(x, residual) -> (residual, normed)``,
              ``forward_rows(x, residual, rows)``; ``as_rms() -> (gain, eps) | None`` (given by the base class:
              None) tells a kernel behind it that it may do the plain RMS formula itself
``mixer``/``ffn`` may return their last product as ``ops.kernels.SliceSums`` (``linear(..., slices_ok=True)``):
              only a norm reads it, and one that says ``TAKES_SLICE_SUMS`` adds the slices itself
``position``  ``prepare(device)``; what it offers (tables) is between it and the mixers that name it
``mixer``     ``cache_spec()`` -> a ``PagedCacheSpec`` (``KVCacheSpec`` or a kind of the mixer's own) | a
              ``SlotCacheSpec`` (``StateSpec``) | ``None``;
              ``forward(x, step, cache, write_cache=True)``
``ffn``       ``forward(x)``; ``forward_after_norm(x, residual, norm) -> (residual, out)`` (given by the base class:
              the norm's ``forward_residual``, then ``forward``) is what a block calls behind its mixer
``block``     ``forward(hidden, residual, step, cache, write_cache) -> (hidden, residual)``
``embedding`` ``forward(token_ids)``
``head``      ``forward(hidden_rows) -> float32 logits``

The reference wires these by hand per model (crates/prelude-core/src/models/qwen3.rs:455-527);
its vocabulary for what a layer keeps between steps is
crates/prelude-core/src/scheduler/components/cache/mod.rs:15-30.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Callable, Dict, Mapping, Optional, Tuple

import torch

# how a tensor is kept on the device and how the random-weights mode draws it
MATRIX = "matrix"   # engine element type; N(0, std)
VECTOR = "vector"   # float32; N(0, std)            (biases)
NORM = "norm"       # float32; 1 + N(0, norm_std)   (norm scales)


@dataclasses.dataclass(frozen=True)
class TensorReq:
    shape: Tuple[int, ...]
    kind: str = MATRIX


class PagedCacheSpec:
    """What a mixer keeps per token, in pages: the interface the cache manager works with.

    A kind of its own is a frozen dataclass derived from this.  Mixers whose specs compare equal share a *group*:
    one pool of pages and one block table per request (each mixer still has its own storage behind those
    tables).  ``window`` > 0 says that a token looks back over that many places only, its own included; pages a
    window has passed are given back while the request lives.  Keys and values (``KVCacheSpec``) are one such
    kind; a mixer that keeps something else per token -- one latent vector, say -- brings its own.
    """
    PAGED = True
    window: int = 0

    def bytes_per_token(self, element_size: int) -> int:
        """Bytes a token takes in this mixer's storage, for an engine element of ``element_size`` bytes."""
        raise NotImplementedError

    def allocate(self, pages: int, page_size: int, dtype: torch.dtype, device: torch.device, group: int):
        """Zeroed storage for ``pages`` pages of ``page_size`` tokens: the object the mixer's ``forward`` gets as
        ``cache``.  It carries ``group``, the index of the step's ``GroupStep`` (block table, slot numbers)."""
        raise NotImplementedError


class SlotCacheSpec:
    """What a mixer keeps per request, of fixed size: a slot of every tensor it names.  ``allocate`` returns the
    object the mixer's ``forward`` gets as ``cache``; it must offer ``zero_fresh(state_slots, fresh)`` (clears the
    rows of starting requests on the device) and, to be replayed from graphs, ``snapshot`` / ``restore``."""
    PAGED = False

    def bytes_per_slot(self) -> int:
        raise NotImplementedError

    def allocate(self, slots: int, device: torch.device):
        raise NotImplementedError


@dataclasses.dataclass
class KVLayerCache:
    """What an attention-like mixer gets: its pages and the group whose tables index them."""
    k: torch.Tensor   # [pages, kv_heads, page_size, head_dim]
    v: torch.Tensor   # [pages, kv_heads, value width (head_dim unless the spec says otherwise), page_size]
    group: int


@dataclasses.dataclass
class StateLayerCache:
    """What a mixer with state of fixed size gets: per name a tensor [slots, *shape]."""
    tensors: Dict[str, torch.Tensor]

    def snapshot(self, state_slots: torch.Tensor) -> Dict[str, torch.Tensor]:
        """Copies of the slots' rows (``state_slots`` int32 on the device, all >= 0)."""
        idx = state_slots.to(torch.int64)
        return {name: t.index_select(0, idx) for name, t in self.tensors.items()}

    def restore(self, state_slots: torch.Tensor, saved: Dict[str, torch.Tensor]) -> None:
        idx = state_slots.to(torch.int64)
        for name, t in self.tensors.items():
            t.index_copy_(0, idx, saved[name])

    def zero_fresh(self, state_slots: torch.Tensor, fresh: torch.Tensor) -> None:
        """Clears the slots of the step's sequences that start their request; both index arrays are the
        step's own on the device, so a captured step can carry this."""
        from ..ops import kernels as K
        for t in self.tensors.values():
            K.zero_fresh_rows(t, state_slots, fresh)


@dataclasses.dataclass(frozen=True)
class KVCacheSpec(PagedCacheSpec):
    """Keys and values per token, in pages.  ``window`` = keys looked back over, own included; 0 = all.
    ``value_dim``: the width of a value where it is not the key's (None: ``head_dim``); mixers with the same
    heads, widths and window share a group of pages.

    Layout per cache slot: K ``[pages, kv_heads, page_size, head_dim]`` and V transposed
    ``[pages, kv_heads, value width, page_size]``, so that both Q.K and P.V read their contraction index
    contiguously (the reference keeps ``[pages, page_size, kv_heads, head_dim]`` for both,
    crates/prelude-core/src/scheduler/components/cache/manager.rs:286-329)."""
    num_kv_heads: int
    head_dim: int
    window: int = 0
    value_dim: Optional[int] = None

    @property
    def v_dim(self) -> int:
        return self.head_dim if self.value_dim is None else self.value_dim

    def bytes_per_token(self, element_size: int) -> int:
        return self.num_kv_heads * (self.head_dim + self.v_dim) * element_size

    def allocate(self, pages, page_size, dtype, device, group):
        return KVLayerCache(torch.zeros((pages, self.num_kv_heads, page_size, self.head_dim), dtype=dtype, device=device),
                            torch.zeros((pages, self.num_kv_heads, self.v_dim, page_size), dtype=dtype, device=device),
                            group)


@dataclasses.dataclass(frozen=True)
class StateSpec(SlotCacheSpec):
    """State of fixed size per request: name -> (shape, element type).  Zeroed when a request starts."""
    tensors: Tuple[Tuple[str, Tuple[int, ...], torch.dtype], ...]

    def bytes_per_slot(self) -> int:
        total = 0
        for _name, shape, dt in self.tensors:
            n = 1
            for d in shape:
                n *= int(d)
            total += n * torch.empty((), dtype=dt).element_size()
        return total

    def allocate(self, slots, device):
        return StateLayerCache({name: torch.zeros((slots, *shape), dtype=dt, device=device)
                                for name, shape, dt in self.tensors})


class Part:
    """Base of all parts.  Subclasses take their sizes and constants as keyword parameters."""

    # False for a part whose ``forward``, in a step of single tokens, reads device results on the host, launches
    # work that depends on them (rows routed by value, say) or works from the step's host-side lists
    # (``StepBatch.q_lens``, ``state_slots_host``): decode steps of a model with such a part are not replayed
    # from HIP graphs.  A part that keeps state per request can be replayed if in such steps it reaches its
    # slots through the device array ``StepBatch.state_slots`` alone; the slots of starting requests are
    # cleared on the device before it runs.
    GRAPH_SAFE = True
    # The same for steps that bring portions of prompts: True says that ``forward`` launches the same work for
    # every step with the same portion lengths, numbers of wanted rows and table width, whatever the tokens, the
    # positions the portions start at, the pages and the state slots are (these it reads on the device).  False
    # by default: a part has to say so itself.
    GRAPH_SAFE_PORTIONS = False
    # Kernel launches one ``forward`` of this part costs the host, about: what a model's parts add up to says up
    # to how many tokens a step with portions is bound by the host's launches and worth replaying from a graph.
    LAUNCHES = 1

    def tensors(self) -> Dict[str, TensorReq]:
        """Local tensor name -> what is required of it."""
        return {}

    def load(self, tensors: Mapping[str, torch.Tensor], dtype: torch.dtype, device: torch.device) -> None:
        """Receives the tensors of ``tensors()`` on the device: MATRIX ones in ``dtype``, others float32."""

    def bind(self, shared: Mapping[str, "Part"]) -> None:
        """Receives the model's shared parts (position encodings) by name, before ``load``."""


class Mixer(Part):
    # True for a mixer that cannot pick a prompt up again where a step left it (nothing carries its state across
    # a cut): the scheduler then feeds a request's known tokens whole in one step or not at all.
    ATOMIC_PREFILL = False

    def cache_spec(self):
        return None

    def forward(self, x: torch.Tensor, step, cache, write_cache: bool = True) -> torch.Tensor:
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError

    def forward_after_norm(self, x, residual, norm: "Norm"):
        """(new residual, forward(norm of residual + x)): what a block asks for behind a mixer.  A feed-forward whose
        first kernel can take the add and the norm in (it learns the norm's kind from ``norm.as_rms()``) does so
        here; this is the plain order."""
        if not norm.TAKES_SLICE_SUMS:
            from ..ops.kernels import as_tensor
            x = as_tensor(x)
        residual, h = norm.forward_residual(x, residual)
        return residual, self.forward(h)


class Norm(Part):
    # True for a norm whose three methods also take a product that was left as partial sums of slices of its
    # inner size (``ops.kernels.SliceSums``) in place of ``x``, adding the slices as it loads them; a block
    # hands other norms the finished tensor.
    TAKES_SLICE_SUMS = False

    def as_rms(self):
        """(gain, eps) if this norm is exactly y = x * rsqrt(mean(x^2) + eps) * gain over the whole row with the
        sum taken of the unrounded residual + x, else None: a kernel that follows may then do the norm itself."""
        return None

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError

    def forward_residual(self, x: torch.Tensor, residual: Optional[torch.Tensor]):
        raise NotImplementedError

    def forward_rows(self, x: torch.Tensor, residual: Optional[torch.Tensor], rows: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class PositionEncoding(Part):
    def prepare(self, device: torch.device) -> None:
        pass


class Block(Part):
    """An arrangement of parts.  ``SLOTS`` names the sub-parts it is built from: slot -> category."""
    SLOTS: Dict[str, str] = {}
    LAUNCHES = 0   # of the arrangement itself; its sub-parts count their own

    def forward(self, hidden, residual, step, cache, write_cache: bool = True):
        raise NotImplementedError

    def launches(self) -> int:
        """Kernel launches of one run of this block: its own and those of the parts in its slots."""
        return self.LAUNCHES + sum(getattr(self, slot).LAUNCHES for slot in self.SLOTS)


# ---------------------------------------------------------------------------
_REGISTRY: Dict[Tuple[str, str], Callable[..., Part]] = {}
CATEGORIES = ("norm", "position", "mixer", "ffn", "block", "embedding", "head")


class PartError(ValueError):
    pass


def register_part(category: str, kind: str):
    """Class decorator: makes ``kind`` buildable in ``category``."""
    if category not in CATEGORIES:
        raise PartError(f"unknown part category {category!r}; one of {CATEGORIES}")

    def deco(cls):
        _REGISTRY[(category, kind)] = cls
        cls.CATEGORY = category
        cls.KIND = kind
        return cls

    return deco


def build_part(category: str, kind: str, params: Mapping[str, Any], **extra) -> Part:
    try:
        cls = _REGISTRY[(category, kind)]
    except KeyError:
        known = sorted(k for c, k in _REGISTRY if c == category)
        raise PartError(f"no {category} of kind {kind!r} is registered (known: {known})") from None
    try:
        return cls(**dict(params), **extra)
    except TypeError as e:
        raise PartError(f"{category} {kind!r} does not take these parameters: {e}") from None


def registered(category: str):
    return sorted(k for c, k in _REGISTRY if c == category)
