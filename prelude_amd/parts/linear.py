"""Embedding and output head.

Embedding rows by token id (crates/prelude-core/src/models/commons/embedding.rs:7-36);
head logits = W h with W [vocab, hidden], the embedding matrix itself when tied
(crates/prelude-core/src/models/qwen3.rs:637-660).  Logits leave in float32.
"""
from __future__ import annotations

import torch

from ..ops import kernels as K
from .base import MATRIX, Part, TensorReq, register_part


@register_part("embedding", "token_embedding")
class TokenEmbedding(Part):
    GRAPH_SAFE_PORTIONS = True   # launches follow the step's shape alone; tokens, positions and pages are read on the device

    def __init__(self, vocab_size: int, hidden_size: int):
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.weight = None

    def tensors(self):
        return {"weight": TensorReq((self.vocab_size, self.hidden_size), MATRIX)}

    def load(self, tensors, dtype, device):
        self.weight = tensors["weight"]

    def forward(self, token_ids: torch.Tensor) -> torch.Tensor:
        return K.embed_gather(token_ids, self.weight)


@register_part("head", "linear_head")
class LinearHead(Part):
    GRAPH_SAFE_PORTIONS = True   # launches follow the step's shape alone; tokens, positions and pages are read on the device

    def __init__(self, vocab_size: int, hidden_size: int):
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.weight = None

    def tensors(self):
        return {"weight": TensorReq((self.vocab_size, self.hidden_size), MATRIX)}

    def load(self, tensors, dtype, device):
        self.weight = K.prepare_weight(tensors["weight"])

    def forward(self, hidden_rows: torch.Tensor) -> torch.Tensor:
        return K.linear(hidden_rows, self.weight, out_dtype=torch.float32)
