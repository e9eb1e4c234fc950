"""Rotary position encoding: the cos/sin tables mixers rotate by.

inv_freq_j = 1 / f32(theta^(2j/d)) with the power in 64-bit, angle
f32(p) * inv_freq_j in 32-bit, cos and sin in 32-bit
(crates/prelude-core/src/models/commons/attn_utils.rs:32-50).  The tables stay
32-bit in every mode (the reference rounds them to the engine's type).
"""
from __future__ import annotations

from typing import Optional

import torch

from .base import PartError, PositionEncoding, register_part


@register_part("position", "rope")
class RotaryEmbedding(PositionEncoding):
    GRAPH_SAFE_PORTIONS = True   # launches follow the step's shape alone; tokens, positions and pages are read on the device

    def __init__(self, rotary_dim: int, max_positions: int, theta: float):
        if rotary_dim <= 0 or rotary_dim % 2:
            raise PartError(f"rope: rotary width {rotary_dim} must be positive and even")
        self.rotary_dim = int(rotary_dim)
        self.max_positions = int(max_positions)
        self.theta = float(theta)
        self.cos: Optional[torch.Tensor] = None
        self.sin: Optional[torch.Tensor] = None

    def prepare(self, device):
        d = self.rotary_dim
        j = torch.arange(0, d, 2, dtype=torch.float64)
        inv_freq = 1.0 / torch.pow(torch.tensor(self.theta, dtype=torch.float64), j / d).to(torch.float32)
        pos = torch.arange(self.max_positions, dtype=torch.float32).reshape(-1, 1)
        ang = pos * inv_freq.reshape(1, -1)
        self.cos = torch.cos(ang).contiguous().to(device)
        self.sin = torch.sin(ang).contiguous().to(device)
