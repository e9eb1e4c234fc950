"""Gated feed-forward: down( act(gate(x)) * up(x) ), no biases.

crates/prelude-core/src/models/qwen3.rs:383-448; silu(x) = x / (1 + e^-x) in
32-bit (crates/prelude-cuda/src/kernels/kernels_src/elementwise/silu_mul.cu:26-33).
Gate and up are one matrix [2I, H] here with rows alternating gate_j, up_j:
one product yields each (gate_j, up_j) pair side by side, so the activation
is the epilogue of that product for few rows and a pairwise kernel otherwise.
The reference's Qwen3 is wired to SiLU whatever ``hidden_act`` says
(qwen3.rs:429-447); the activation is a parameter here (SiLU, or GELU in its
tanh form: crates/prelude-core/src/models/commons/activation.rs:3-25), one
epilogue code in the same kernels.
"""
from __future__ import annotations

import torch

from ..ops import kernels as K
from .base import MATRIX, FeedForward, PartError, TensorReq, register_part


@register_part("ffn", "gated_mlp")
class GatedMLP(FeedForward):
    LAUNCHES = 3   # gate and up in one product, activation * up, down
    GRAPH_SAFE_PORTIONS = True   # launches follow the step's shape alone; tokens, positions and pages are read on the device

    def __init__(self, hidden_size: int, intermediate_size: int, activation: str = "silu"):
        if activation not in K.GATE_ACTIVATIONS:
            raise PartError(f"gated_mlp: activation {activation!r} is not one of {sorted(K.GATE_ACTIVATIONS)}")
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)
        self.activation = activation
        self.gate_up = None
        self.down = None

    def tensors(self):
        h, i = self.hidden_size, self.intermediate_size
        return {"gate_proj.weight": TensorReq((i, h), MATRIX), "up_proj.weight": TensorReq((i, h), MATRIX),
                "down_proj.weight": TensorReq((h, i), MATRIX)}

    def load(self, tensors, dtype, device):
        g, u = tensors["gate_proj.weight"], tensors["up_proj.weight"]
        self.gate_up = K.prepare_weight(
            torch.stack([g, u], dim=1).reshape(2 * self.intermediate_size, self.hidden_size).contiguous())
        self.down = K.prepare_weight(tensors["down_proj.weight"])

    def forward(self, x):
        return K.linear(K.linear_gated(x, self.gate_up, self.activation), self.down, slices_ok=True)

    def forward_after_norm(self, x, residual, norm):
        # a few rows behind an RMS norm: the add and the norm ride in the gated product's staging of X
        rms = norm.as_rms() if residual is not None else None
        if rms is None or not K.gated_after_norm_supported(x, residual, self.gate_up, self.activation):
            return super().forward_after_norm(x, residual, norm)
        residual, h = K.linear_gated_after_norm(x, residual, rms[0], rms[1], self.gate_up, self.activation)
        return residual, K.linear(h, self.down, slices_ok=True)
