"""RMSNorm, alone or fused with the residual add.

y = x * rsqrt(mean(x^2) + eps) * w in 32-bit
(crates/prelude-core/src/models/commons/linear.rs:435-501); with a residual:
sum in 32-bit, the residual keeps the rounded sum, the norm is taken of the
unrounded one (crates/prelude-cuda/src/kernels/kernels_src/normalization/rmsnorm.cu:258-274).
"""
from __future__ import annotations

from typing import Optional

import torch

from ..ops import kernels as K
from .base import NORM, Norm, TensorReq, register_part


@register_part("norm", "rms_norm")
class RMSNorm(Norm):
    GRAPH_SAFE_PORTIONS = True   # launches follow the step's shape alone; tokens, positions and pages are read on the device

    TAKES_SLICE_SUMS = True

    def __init__(self, size: int, eps: float):
        self.size = int(size)
        self.eps = float(eps)
        self.weight: Optional[torch.Tensor] = None

    def tensors(self):
        return {"weight": TensorReq((self.size,), NORM)}

    def load(self, tensors, dtype, device):
        self.weight = tensors["weight"]

    def as_rms(self):
        return self.weight, self.eps

    def forward(self, x):
        return K.rmsnorm(x, self.weight, self.eps)

    def forward_residual(self, x, residual):
        """First use in a model: residual None -> (x, norm(x)).  Afterwards the
        residual is updated in place with residual + x."""
        if residual is None:
            x = K.as_tensor(x)
            return x, K.rmsnorm(x, self.weight, self.eps)
        out = K.rmsnorm(x, self.weight, self.eps, residual=residual)
        return residual, out

    def forward_rows(self, x, residual, rows):
        return K.rmsnorm(x, self.weight, self.eps, residual=residual, rows=rows)
