"""Arrangements of parts into one layer.

``prenorm``: norm -> mixer -> (+residual) norm -> feed-forward, with the
residual carried beside the hidden state and each add deferred into the next
norm (crates/prelude-core/src/models/qwen3.rs:486-502,
crates/prelude-core/src/models/commons/linear.rs:471-488).
"""
from __future__ import annotations

from ..ops import kernels as K
from .base import Block, register_part


@register_part("block", "prenorm")
class PreNormBlock(Block):
    GRAPH_SAFE_PORTIONS = True   # launches follow the step's shape alone; tokens, positions and pages are read on the device

    SLOTS = {"input_norm": "norm", "mixer": "mixer", "post_mixer_norm": "norm", "ffn": "ffn"}

    def __init__(self, input_norm, mixer, post_mixer_norm, ffn):
        self.input_norm, self.mixer, self.post_mixer_norm, self.ffn = input_norm, mixer, post_mixer_norm, ffn

    def forward(self, hidden, residual, step, cache, write_cache=True):
        # a mixer's or feed-forward's last product may come as partial sums of slices (``K.SliceSums``): a norm
        # that can adds them as it loads them, any other gets the finished tensor
        if not self.input_norm.TAKES_SLICE_SUMS:
            hidden = K.as_tensor(hidden)
        residual, h = self.input_norm.forward_residual(hidden, residual)
        h = self.mixer.forward(h, step, cache, write_cache)
        residual, h = self.ffn.forward_after_norm(h, residual, self.post_mixer_norm)
        return h, residual
