"""Grouped-query attention over a paged cache, with optional per-head QK norm,
rotary encoding, biases and a window.

One merged projection [(nh + 2 nkv) hd, H] (crates/prelude-core/src/models/qwen3.rs:89-106,
crates/prelude-core/src/models/commons/attn_utils.rs:91-133; unlike the
reference's merged path, biases are kept), per-head RMSNorm of q and k with a
weight shared by all heads and RoPE straight after it
(qwen3.rs:59-62, :175-186), K and V written to the cache, causal softmax
attention with scale 1/sqrt(head_dim) (qwen3.rs:126, :191-206), output
projection (qwen3.rs:226-228).
"""
from __future__ import annotations

import math
from typing import Optional

import torch

from ..ops import kernels as K
from .base import MATRIX, NORM, VECTOR, KVCacheSpec, Mixer, PartError, TensorReq, register_part


@register_part("mixer", "gqa_attention")
class GQAAttention(Mixer):
    LAUNCHES = 4   # merged projection, norm + rotation + cache write, attention, output projection
    GRAPH_SAFE_PORTIONS = True   # launches follow the step's shape alone; tokens, positions and pages are read on the device

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, norm_eps: float = 1e-6,
                 qk_norm: bool = True, bias: bool = False, window: int = 0, position: Optional[str] = None,
                 rotary_dim: Optional[int] = None, scale: Optional[float] = None, score_cap: float = 0.0):
        if num_heads % num_kv_heads:
            raise PartError(f"gqa_attention: {num_heads} heads are not a multiple of {num_kv_heads} KV heads")
        # what the kernels take: the matrix-core attention has head sizes of its own (others go to the generic
        # kernel), the generic kernel and the norm + rotation kernel any size up to 256
        if not 1 <= head_dim <= 256:
            raise PartError(f"gqa_attention: head_dim {head_dim} is outside 1..256")
        self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim = hidden_size, num_heads, num_kv_heads, head_dim
        self.norm_eps, self.qk_norm, self.bias, self.window = float(norm_eps), bool(qk_norm), bool(bias), int(window or 0)
        self.position = position
        self.rotary_dim = (head_dim if rotary_dim is None else int(rotary_dim)) if position else 0
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        # > 0: scaled scores are bent to cap * tanh(score / cap) before the softmax (the reference's Qwen3 has none,
        # qwen3.rs:204; a parameter for mixers of other models)
        self.score_cap = float(score_cap or 0.0)
        if self.score_cap < 0:
            raise PartError(f"gqa_attention: a score cap of {score_cap} is negative")
        self.rope = None
        self.w_qkv = self.b_qkv = self.w_o = self.b_o = self.q_norm = self.k_norm = None

    def cache_spec(self):
        return KVCacheSpec(self.num_kv_heads, self.head_dim, self.window)

    def bind(self, shared):
        if self.position is not None:
            if self.position not in shared:
                raise PartError(f"gqa_attention: the model has no position encoding named {self.position!r}")
            self.rope = shared[self.position]
            if getattr(self.rope, "rotary_dim", None) != self.rotary_dim:
                raise PartError(f"gqa_attention: position encoding {self.position!r} has width "
                                f"{getattr(self.rope, 'rotary_dim', None)}, the mixer rotates {self.rotary_dim}")

    def tensors(self):
        h, nh, nkv, hd = self.hidden_size, self.num_heads, self.num_kv_heads, self.head_dim
        t = {"q_proj.weight": TensorReq((nh * hd, h), MATRIX), "k_proj.weight": TensorReq((nkv * hd, h), MATRIX),
             "v_proj.weight": TensorReq((nkv * hd, h), MATRIX), "o_proj.weight": TensorReq((h, nh * hd), MATRIX)}
        if self.bias:
            t.update({"q_proj.bias": TensorReq((nh * hd,), VECTOR), "k_proj.bias": TensorReq((nkv * hd,), VECTOR),
                      "v_proj.bias": TensorReq((nkv * hd,), VECTOR), "o_proj.bias": TensorReq((h,), VECTOR)})
        if self.qk_norm:
            t.update({"q_norm.weight": TensorReq((hd,), NORM), "k_norm.weight": TensorReq((hd,), NORM)})
        return t

    def load(self, tensors, dtype, device):
        self.w_qkv = K.prepare_weight(torch.cat([tensors["q_proj.weight"], tensors["k_proj.weight"],
                                                 tensors["v_proj.weight"]], dim=0).contiguous())
        self.w_o = K.prepare_weight(tensors["o_proj.weight"])
        if self.bias:
            self.b_qkv = torch.cat([tensors["q_proj.bias"], tensors["k_proj.bias"], tensors["v_proj.bias"]]).contiguous()
            self.b_o = tensors["o_proj.bias"]
        if self.qk_norm:
            self.q_norm, self.k_norm = tensors["q_norm.weight"], tensors["k_norm.weight"]

    FUSED_DECODE_MAX_SEQS = 256   # measured: +3 % tokens a second at batch 1, +1 to 2 % at 8, 16, 32 and 64

    def _fused_decode(self, x, step, cache) -> bool:
        """Few sequences, each feeding one token: a kernel less per layer counts for more than the norm and the
        rotation that every workgroup of the attention kernel then does for itself."""
        return (x.dtype == torch.bfloat16 and self.rope is not None and step.decode_seqs is not None
                and step.n_prefill == 0 and step.n_decode == step.num_seqs <= self.FUSED_DECODE_MAX_SEQS
                and K.attention_decode_fused_supported(self.num_heads, self.num_kv_heads, self.head_dim,
                                                       self.rotary_dim, cache.k.shape[2]))

    def forward(self, x, step, cache, write_cache=True):
        nh, nkv, hd = self.num_heads, self.num_kv_heads, self.head_dim
        g = step.kv[cache.group]
        cos = self.rope.cos if self.rope is not None else None
        sin = self.rope.sin if self.rope is not None else None
        if write_cache and self._fused_decode(x, step, cache):
            # a step of single tokens: the norm, the rotation and the cache write happen inside the attention kernel
            qkv = K.linear(x, self.w_qkv, self.b_qkv)
            o = K.attention_decode_fused(qkv, self.q_norm, self.k_norm, cos, sin, g.slots, self.norm_eps,
                                         cache.k, cache.v, g.block_table, step.decode_seqs, step.cu_q, step.context_lens,
                                         nh, step.max_decode_context, self.window, self.scale, every_seq=True,
                                         softcap=self.score_cap)
            return K.linear(o.view(o.shape[0], nh * hd), self.w_o, self.b_o, slices_ok=True)
        if write_cache:
            qkv = K.linear(x, self.w_qkv, self.b_qkv)
            q = K.qknorm_rope_kv(qkv, self.q_norm, self.k_norm, cos, sin, step.positions, g.slots, cache.k, cache.v,
                                 nh, nkv, hd, self.rotary_dim, self.norm_eps)
        else:  # reads keys and values another layer wrote: only the queries are projected
            bq = self.b_qkv[: nh * hd] if self.b_qkv is not None else None
            qx = K.linear(x, self.w_qkv.first_rows(nh * hd), bq)
            q = K.qknorm_rope_kv(qx, self.q_norm, None, cos, sin, step.positions, None, None, None, nh, 0, hd,
                                 self.rotary_dim, self.norm_eps)
        o = K.attention(q, cache.k, cache.v, g, step, self.window, self.scale, self.score_cap)
        return K.linear(o.view(o.shape[0], nh * hd), self.w_o, self.b_o, slices_ok=True)
