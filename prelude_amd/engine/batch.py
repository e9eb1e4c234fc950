"""What one step brings to the model: the tokens of every portion, as one packed batch.

The reference builds the same arrays per step
(crates/prelude-core/src/engine/model_runner/paged_mixed.rs:32-117: packed
tokens, positions, cumulative query lengths, block tables, slot mapping) and
uploads them one by one; here they travel in a single int32 buffer.
"""
from __future__ import annotations

import dataclasses
from typing import List, Optional

import torch


@dataclasses.dataclass
class GroupStep:
    """Per cache group: where each sequence's pages are and where each token's key goes."""
    block_table: torch.Tensor  # int32 [B, stride], -1 = no page (padding or given back)
    slots: torch.Tensor        # int32 [T], page * page_size + offset


@dataclasses.dataclass
class StepBatch:
    num_tokens: int
    num_seqs: int
    token_ids: torch.Tensor      # int32 [T]
    positions: torch.Tensor      # int32 [T] absolute position of each token
    seq_of_token: torch.Tensor   # int32 [T] index of the portion a token belongs to
    cu_q: torch.Tensor           # int32 [B + 1] prefix sums of portion lengths
    context_lens: torch.Tensor   # int32 [B] tokens in the cache after this step
    state_slots: torch.Tensor    # int32 [B] slot of per-request state, -1 if none
    fresh: torch.Tensor          # int32 [B] 1 when the portion starts its request (state must start from zero)
    want_rows: torch.Tensor      # int32 [W] packed token rows whose logits are wanted
    kv: List[GroupStep]
    # host copies for decisions that must not wait for the device
    q_lens: List[int] = dataclasses.field(default_factory=list)
    starts: List[int] = dataclasses.field(default_factory=list)
    state_slots_host: List[int] = dataclasses.field(default_factory=list)
    fresh_host: List[int] = dataclasses.field(default_factory=list)
    max_q_len: int = 0
    max_context_len: int = 0
    # the step's sequences by kind, for kernels that treat single tokens and portions differently
    decode_seqs: Optional[torch.Tensor] = None    # int32 [n_decode] indices of sequences feeding one token
    prefill_seqs: Optional[torch.Tensor] = None   # int32 [n_prefill] indices of sequences feeding more
    n_decode: int = 0
    n_prefill: int = 0
    max_prefill_q: int = 0       # longest portion among prefill_seqs
    min_prefill_prefix: int = 0  # fewest tokens any of prefill_seqs has behind it already
    max_decode_context: int = 0  # longest context among decode_seqs
    page_size: int = 0
    graph: Optional[object] = None  # set while a step is being captured or replayed from fixed buffers

    @property
    def all_decode(self) -> bool:
        return self.max_q_len == 1
