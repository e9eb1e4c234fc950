"""A plain, slow implementation of the Qwen3 dense decoder for whole sequences.

No cache, no batching, no kernels: one function per part, written from the
formulas of Virtue-Research/prelude (cited per function as file:line relative
to the reference root).  It shares no code with ``prelude_amd``: it takes a
dict of config.json keys and a dict of tensors by safetensors name.

Everything is computed in ``dtype`` (float64 by default, so that the plain
implementation's own rounding does not blur a comparison with a 32-bit
engine; float32 gives the arithmetic the reference itself uses).
"""
from __future__ import annotations

import math

import torch


# --------------------------------------------------------------------------
# parts
# --------------------------------------------------------------------------
def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """y = x * rsqrt(mean(x^2) + eps) * w over the last axis.

    crates/prelude-core/src/models/commons/linear.rs:491-500 (Module::forward)
    and crates/prelude-cuda/src/kernels/kernels_src/normalization/rmsnorm.cu:36-51.
    """
    var = (x * x).mean(dim=-1, keepdim=True)
    return x * torch.rsqrt(var + eps) * weight


def rope_tables(head_dim: int, max_pos: int, theta: float, dtype=torch.float64):
    """cos/sin tables [max_pos, head_dim/2].

    crates/prelude-core/src/models/commons/attn_utils.rs:32-50:
    inv_freq_j = 1 / f32(theta^(2j/hd)) with the power in f64, the angle
    f32(p) * inv_freq_j in f32, cos/sin in f32.  The angle is kept in float32
    here whatever ``dtype`` is, because that rounding is part of the formula
    (it changes the angle by up to p * 2^-24, far more than later rounding).
    """
    j = torch.arange(0, head_dim, 2, dtype=torch.float64)
    inv_freq = (1.0 / torch.tensor(theta, dtype=torch.float64).pow(j / head_dim).to(torch.float32)).to(torch.float32)
    pos = torch.arange(max_pos, dtype=torch.float32).reshape(max_pos, 1)
    ang = pos * inv_freq.reshape(1, -1)  # float32 product
    if dtype == torch.float64:
        # cos/sin of the float32 angle, evaluated exactly
        return torch.cos(ang.double()), torch.sin(ang.double())
    return torch.cos(ang).to(dtype), torch.sin(ang).to(dtype)


def apply_rope(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """Rotate-half over the whole head width.

    x [S, heads, hd], cos/sin [S, hd/2] (already gathered at the positions).
    out[j] = x[j] cos[j] - x[j+hd/2] sin[j]; out[j+hd/2] = x[j+hd/2] cos[j] + x[j] sin[j].
    crates/prelude-core/src/models/commons/attn_utils.rs:52-59;
    crates/prelude-cuda/src/kernels/kernels_src/rope/qknorm_rope.cu:67-90.
    """
    half = x.shape[-1] // 2
    x1, x2 = x[..., :half], x[..., half:]
    c, s = cos[:, None, :], sin[:, None, :]
    return torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], dim=-1)


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float,
              window: int | None = None, q_offset: int = 0) -> torch.Tensor:
    """Causal softmax attention with grouped heads, by explicit loops over heads.

    q [Sq, nh, hd], k/v [Sk, nkv, hd]; query row r has absolute position
    q_offset + r and sees keys c <= q_offset + r (and, with a window of W
    keys, c > q_offset + r - W).  Query head h reads KV head h // (nh/nkv).
    crates/prelude-core/src/models/qwen3.rs:276-370 (matmul_cross_attention),
    crates/prelude-core/src/ops/traits/attention.rs:10-99 (mask, incl.
    SlidingWindow{left = W-1}; crates/prelude-core/src/models/gemma3.rs:298-301).
    """
    sq, nh, hd = q.shape
    sk, nkv, _ = k.shape
    group = nh // nkv
    out = torch.empty_like(q)
    qi = torch.arange(sq).reshape(sq, 1) + q_offset
    ki = torch.arange(sk).reshape(1, sk)
    allowed = ki <= qi
    if window is not None:
        allowed &= ki > qi - window
    for h in range(nh):
        kh = k[:, h // group, :]
        vh = v[:, h // group, :]
        scores = (q[:, h, :] @ kh.T) * scale
        scores = scores.masked_fill(~allowed, float("-inf"))
        out[:, h, :] = torch.softmax(scores, dim=-1) @ vh
    return out


def silu(x: torch.Tensor) -> torch.Tensor:
    """x / (1 + exp(-x)). crates/prelude-cuda/src/kernels/kernels_src/common/common.cuh:78-80."""
    return x / (1.0 + torch.exp(-x))


def swiglu(x, w_gate, w_up, w_down):
    """down( silu(gate(x)) * up(x) ), no biases. crates/prelude-core/src/models/qwen3.rs:429-447."""
    return (silu(x @ w_gate.T) * (x @ w_up.T)) @ w_down.T


def linear(x, w, b=None):
    """y = x W^T (+ b), W [out, in]. crates/prelude-core/src/models/commons/linear.rs:30-98."""
    y = x @ w.T
    return y if b is None else y + b


# --------------------------------------------------------------------------
# which layers have a window
# --------------------------------------------------------------------------
def layer_window(cfg: dict, i: int) -> int | None:
    """The reference refuses use_sliding_window (crates/prelude-core/src/models/qwen3.rs:50-52).

    This build reads the three keys the reference parses
    (crates/prelude-core/src/models/config.rs:14-20) as: with
    ``use_sliding_window`` true, layers with index >= ``max_window_layers``
    attend to the last ``sliding_window`` keys (the query's own included).
    """
    if cfg.get("use_sliding_window") and cfg.get("sliding_window") and i >= cfg["max_window_layers"]:
        return int(cfg["sliding_window"])
    return None


# --------------------------------------------------------------------------
# the whole model
# --------------------------------------------------------------------------
def attention_block(cfg: dict, w: dict, i: int, h: torch.Tensor, cos, sin) -> torch.Tensor:
    """q/k/v projection, per-head QK-RMSNorm, RoPE, attention, output projection.

    crates/prelude-core/src/models/qwen3.rs:161-231; the norm over head_dim
    with a weight shared by all heads and the layer's eps: qwen3.rs:59-62,
    :120, :175-186; scale 1/sqrt(head_dim): qwen3.rs:126.
    """
    p = f"model.layers.{i}.self_attn."
    nh, nkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    s = h.shape[0]
    bias = cfg["attention_bias"]
    q = linear(h, w[p + "q_proj.weight"], w[p + "q_proj.bias"] if bias else None).reshape(s, nh, hd)
    k = linear(h, w[p + "k_proj.weight"], w[p + "k_proj.bias"] if bias else None).reshape(s, nkv, hd)
    v = linear(h, w[p + "v_proj.weight"], w[p + "v_proj.bias"] if bias else None).reshape(s, nkv, hd)
    q = rms_norm(q, w[p + "q_norm.weight"], cfg["rms_norm_eps"])
    k = rms_norm(k, w[p + "k_norm.weight"], cfg["rms_norm_eps"])
    q = apply_rope(q, cos, sin)
    k = apply_rope(k, cos, sin)
    o = attention(q, k, v, 1.0 / math.sqrt(hd), window=layer_window(cfg, i))
    return linear(o.reshape(s, nh * hd), w[p + "o_proj.weight"], w[p + "o_proj.bias"] if bias else None)


def forward(cfg: dict, weights: dict, tokens, dtype=torch.float64, position_offset: int = 0) -> torch.Tensor:
    """Logits [S, V] for every position of one whole sequence (token r stands
    at position position_offset + r; only used to test the shift invariance).

    Pre-norm blocks with the residual carried beside the hidden state:
    crates/prelude-core/src/models/qwen3.rs:486-502, :601-623 and
    crates/prelude-core/src/models/commons/linear.rs:471-488; written here
    in the equivalent plain form x += attn(norm(x)); x += mlp(norm(x)).
    Head: crates/prelude-core/src/models/qwen3.rs:637-660 (tied: the embedding
    matrix itself).
    """
    w = {k: v.to(dtype) for k, v in weights.items()}
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    s = tokens.shape[0]
    eps = cfg["rms_norm_eps"]
    cos_t, sin_t = rope_tables(cfg["head_dim"], cfg["max_position_embeddings"], cfg["rope_theta"], dtype)
    cos, sin = cos_t[position_offset:position_offset + s], sin_t[position_offset:position_offset + s]
    x = w["model.embed_tokens.weight"][tokens]
    for i in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{i}."
        h = rms_norm(x, w[p + "input_layernorm.weight"], eps)
        x = x + attention_block(cfg, w, i, h, cos, sin)
        h = rms_norm(x, w[p + "post_attention_layernorm.weight"], eps)
        x = x + swiglu(h, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], w[p + "mlp.down_proj.weight"])
    x = rms_norm(x, w["model.norm.weight"], eps)
    head = w["model.embed_tokens.weight"] if cfg["tie_word_embeddings"] else w["lm_head.weight"]
    return x @ head.T


def greedy(cfg: dict, weights: dict, prompt, n: int, dtype=torch.float64) -> list[int]:
    """n greedy tokens by re-running the whole sequence each time
    (crates/prelude-core/src/models/qwen3.rs:1038-1092 tests the same thing);
    ties go to the lowest index (crates/prelude-cuda/src/kernels/kernels_src/sample/fast_argmax_vocab.cu:38-47).
    """
    seq = list(prompt)
    out = []
    for _ in range(n):
        logits = forward(cfg, weights, seq, dtype)[-1]
        t = int(torch.argmax(logits))  # torch returns the first maximal index
        out.append(t)
        seq.append(t)
    return out


# --------------------------------------------------------------------------
# sampling
# --------------------------------------------------------------------------
def sampling_probs(logits: torch.Tensor, temperature: float, top_k: int | None = None,
                   top_p: float | None = None) -> torch.Tensor:
    """The distribution the reference draws from: softmax(logits / T), then
    top-k (keep the k largest), then top-p (sorted descending, keep while the
    mass before an entry is < p), not renormalised (a weighted draw follows).
    crates/prelude-core/src/engine/sampling/logits_processor.rs:51-136.
    """
    prs = torch.softmax(logits.double() / temperature, dim=-1)
    if top_k is not None and 0 < top_k < prs.numel():
        kth = torch.topk(prs, top_k).values[-1]
        prs = torch.where(prs >= kth, prs, torch.zeros_like(prs))
    if top_p is not None and 0.0 < top_p < 1.0:
        order = torch.argsort(prs, descending=True, stable=True)
        cum = 0.0
        keep = torch.zeros_like(prs)
        for idx in order.tolist():
            if cum >= top_p:
                break
            keep[idx] = prs[idx]
            cum += float(prs[idx])
        prs = keep
    return prs


def draw(prs: torch.Tensor, u: float) -> int:
    """Inverse-CDF draw: the first index whose cumulative weight exceeds u * total."""
    cdf = torch.cumsum(prs.double(), dim=0)
    target = u * float(cdf[-1])
    idx = int(torch.searchsorted(cdf, torch.tensor(target, dtype=torch.float64), right=True))
    return min(idx, prs.numel() - 1)


# --------------------------------------------------------------------------
# tiny configurations and random weights
# --------------------------------------------------------------------------
def tiny_config_a() -> dict:
    return dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=256, hidden_size=64,
                intermediate_size=128, num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2,
                head_dim=16, attention_bias=False, max_position_embeddings=128, sliding_window=None,
                max_window_layers=2, tie_word_embeddings=True, rope_theta=10000.0, rms_norm_eps=1e-6,
                use_sliding_window=False, hidden_act="silu", eos_token_id=255)


def tiny_config_b() -> dict:
    return dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=509, hidden_size=96,
                intermediate_size=160, num_hidden_layers=3, num_attention_heads=6, num_key_value_heads=1,
                head_dim=32, attention_bias=False, max_position_embeddings=256, sliding_window=None,
                max_window_layers=3, tie_word_embeddings=False, rope_theta=1000000.0, rms_norm_eps=1e-5,
                use_sliding_window=False, hidden_act="silu", eos_token_id=[507, 508])


def tiny_config_c() -> dict:
    """Differs from A and B again: three query heads per KV head, head_dim 48,
    biases, and a window of 24 keys on the upper two of four layers."""
    return dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=331, hidden_size=80,
                intermediate_size=112, num_hidden_layers=4, num_attention_heads=6, num_key_value_heads=2,
                head_dim=48, attention_bias=True, max_position_embeddings=512, sliding_window=24,
                max_window_layers=2, tie_word_embeddings=False, rope_theta=50000.0, rms_norm_eps=3e-6,
                use_sliding_window=True, hidden_act="silu", eos_token_id=330)


def tensor_shapes(cfg: dict) -> dict:
    """Every tensor a Qwen3ForCausalLM checkpoint holds, by name
    (crates/prelude-core/src/models/qwen3.rs:59-81, :112-117, :392-409, :469-477, :545-565, :639-643)."""
    h, i, v = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    nh, nkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    shapes = {"model.embed_tokens.weight": (v, h), "model.norm.weight": (h,)}
    if not cfg["tie_word_embeddings"]:
        shapes["lm_head.weight"] = (v, h)
    for l in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{l}."
        shapes[p + "input_layernorm.weight"] = (h,)
        shapes[p + "post_attention_layernorm.weight"] = (h,)
        shapes[p + "self_attn.q_proj.weight"] = (nh * hd, h)
        shapes[p + "self_attn.k_proj.weight"] = (nkv * hd, h)
        shapes[p + "self_attn.v_proj.weight"] = (nkv * hd, h)
        shapes[p + "self_attn.o_proj.weight"] = (h, nh * hd)
        shapes[p + "self_attn.q_norm.weight"] = (hd,)
        shapes[p + "self_attn.k_norm.weight"] = (hd,)
        if cfg["attention_bias"]:
            shapes[p + "self_attn.q_proj.bias"] = (nh * hd,)
            shapes[p + "self_attn.k_proj.bias"] = (nkv * hd,)
            shapes[p + "self_attn.v_proj.bias"] = (nkv * hd,)
            shapes[p + "self_attn.o_proj.bias"] = (h,)
        shapes[p + "mlp.gate_proj.weight"] = (i, h)
        shapes[p + "mlp.up_proj.weight"] = (i, h)
        shapes[p + "mlp.down_proj.weight"] = (h, i)
    return shapes


def random_weights(cfg: dict, seed: int, std: float = 0.02, norm_std: float = 0.01,
                   dtype=torch.float32) -> dict:
    """Matrices and biases N(0, std), norm weights 1 + N(0, norm_std); the test
    suite's own generator (the engine's random-weights mode is a separate one)."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in sorted(tensor_shapes(cfg).items()):
        t = torch.randn(shape, generator=g, dtype=torch.float32)
        if name.endswith("norm.weight") or "layernorm" in name:
            t = 1.0 + norm_std * t
        else:
            t = std * t
        out[name] = t.to(dtype)
    return out
