"""A model as data: which parts each layer is made of, in which order layers
run, and which cache each run uses.

Nothing here computes.  An architecture turns its typed configuration into a
``ModelSpec``; ``prelude_amd.models.causal_lm.CausalLM`` builds the parts from
the registry, asks them for their tensors, and runs them.
"""
from __future__ import annotations

import dataclasses
from typing import Any, Dict, List, Optional, Tuple


@dataclasses.dataclass
class PartSpec:
    kind: str                                   # registry key within the part's category
    params: Dict[str, Any] = dataclasses.field(default_factory=dict)   # sizes and constants
    weights: Dict[str, str] = dataclasses.field(default_factory=dict)  # local tensor name -> checkpoint name


@dataclasses.dataclass
class LayerSpec:
    block: str                                  # arrangement kind, e.g. "prenorm"
    parts: Dict[str, PartSpec]                  # the block's slots, e.g. input_norm / mixer / post_mixer_norm / ffn
    block_params: Dict[str, Any] = dataclasses.field(default_factory=dict)


@dataclasses.dataclass
class RunSpec:
    """One entry of the order in which layers run.

    ``layer`` may appear in several runs (the same weights applied again).
    Each run has a cache of its own unless ``reads_cache_of`` names an earlier
    run (by its index in ``order``) whose cache it reads without writing.
    """
    layer: int
    reads_cache_of: Optional[int] = None


@dataclasses.dataclass
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    max_positions: int
    eos_token_ids: Tuple[int, ...]
    embedding: PartSpec
    layers: List[LayerSpec]
    order: List[RunSpec]
    final_norm: PartSpec
    head: PartSpec
    positions: Dict[str, PartSpec] = dataclasses.field(default_factory=dict)  # shared position encodings by name
    # checkpoint names (shell patterns) that files of this architecture may hold and the model does not read:
    # they are passed over; any other tensor nothing asks for is an error
    ignored_tensors: Tuple[str, ...] = ()

    def validate(self) -> None:
        if not self.order:
            raise ValueError("model spec: the run order is empty")
        for i, r in enumerate(self.order):
            if not 0 <= r.layer < len(self.layers):
                raise ValueError(f"model spec: run {i} names layer {r.layer}, there are {len(self.layers)}")
            if r.reads_cache_of is not None:
                if not 0 <= r.reads_cache_of < i:
                    raise ValueError(f"model spec: run {i} reads the cache of run {r.reads_cache_of}, "
                                     f"which does not come before it")
                if self.order[r.reads_cache_of].reads_cache_of is not None:
                    raise ValueError(f"model spec: run {i} reads the cache of run {r.reads_cache_of}, "
                                     f"which has none of its own")
