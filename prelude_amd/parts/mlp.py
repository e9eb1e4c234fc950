"""Gated feed-forward: down( act(gate(x)) * up(x) ), no biases.

crates/prelude-core/src/models/qwen3.rs:383-448; silu(x) = x / (1 + e^-x) in
32-bit (crates/prelude-cuda/src/kernels/kernels_src/elementwise/silu_mul.cu:26-33).
Gate and up are one matrix [2I, H] here, gate rows first, so one product feeds
the activation kernel.
"""
from __future__ import annotations

import torch

from ..ops import kernels as K
from .base import MATRIX, FeedForward, PartError, TensorReq, register_part


@register_part("ffn", "gated_mlp")
class GatedMLP(FeedForward):
    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "silu"):
        if activation != "silu":
            raise PartError(f"gated_mlp: activation {activation!r} is not supported (silu)")
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.gate_up = None
        self.down = None

    def tensors(self):
        h, i = self.hidden_size, self.intermediate_size
        return {"gate_proj.weight": TensorReq((i, h), MATRIX), "up_proj.weight": TensorReq((i, h), MATRIX),
                "down_proj.weight": TensorReq((h, i), MATRIX)}

    def load(self, tensors, dtype, device):
        self.gate_up = torch.cat([tensors["gate_proj.weight"], tensors["up_proj.weight"]], dim=0).contiguous()
        self.down = tensors["down_proj.weight"]

    def forward(self, x):
        return K.linear(K.silu_mul(K.linear(x, self.gate_up)), self.down)
