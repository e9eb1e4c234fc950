"""What every part of a layer is, and the registry parts are built from.

A model is described as data (``prelude_amd.models.spec``): each layer names
its parts by *kind* with their sizes and constants as parameters.  A part
knows nothing of the model it sits in: it gets its parameters, says which
tensors it needs (by local name and shape), receives them, and runs.

Categories and the interface each must have:

``norm``      ``forward(x)``, ``forward_residual(x, residual) -> (residual, normed)``,
              ``forward_rows(x, residual, rows)``
``mixer``/``ffn`` may return their last product as ``ops.kernels.SliceSums`` (``linear(..., slices_ok=True)``):
              only a norm reads it, and one that says ``TAKES_SLICE_SUMS`` adds the slices itself
``position``  ``prepare(device)``; what it offers (tables) is between it and the mixers that name it
``mixer``     ``cache_spec()`` -> ``KVCacheSpec`` | ``StateSpec`` | ``None``;
              ``forward(x, step, cache, write_cache=True)``
``ffn``       ``forward(x)``
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


@dataclasses.dataclass(frozen=True)
class KVCacheSpec:
    """Keys and values per token, in pages.  ``window`` = keys looked back over, own included; 0 = all.
    ``value_dim``: the width of a value where it is not the key's (None: ``head_dim``); mixers with the same
    heads, widths and window share a group of pages."""
    num_kv_heads: int
    head_dim: int
    window: int = 0
    value_dim: Optional[int] = None

    @property
    def v_dim(self) -> int:
        return self.head_dim if self.value_dim is None else self.value_dim


@dataclasses.dataclass(frozen=True)
class StateSpec:
    """State of fixed size per request: name -> (shape, element type).  Zeroed when a request starts."""
    tensors: Tuple[Tuple[str, Tuple[int, ...], torch.dtype], ...]


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


class Norm(Part):
    # True for a norm whose three methods also take a product that was left as partial sums of slices of its
    # inner size (``ops.kernels.SliceSums``) in place of ``x``, adding the slices as it loads them; a block
    # hands other norms the finished tensor.
    TAKES_SLICE_SUMS = False

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

    def forward(self, hidden, residual, step, cache, write_cache: bool = True):
        raise NotImplementedError


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
