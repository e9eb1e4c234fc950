"""Qwen3 dense: from its typed configuration to a model specification.

Decoder with grouped-query attention, per-head QK-RMSNorm, RoPE over the whole
head, SwiGLU feed-forward, pre-norm RMSNorm, tied or separate output head
(crates/prelude-core/src/models/qwen3.rs:24-660); tensor names as read there
(:59-81, :112-117, :392-409, :469-477, :545-565, :639-643); registry entry
(:1097-1237: aliases "Qwen3"/"Qwen3Model", model_type "qwen3").
"""
from __future__ import annotations

from ..config.model_config import ConfigError, Qwen3Config
from ..config.registry import Architecture, register_architecture
from .spec import LayerSpec, ModelSpec, PartSpec, RunSpec


def qwen3_spec(cfg: Qwen3Config) -> ModelSpec:
    if cfg.hidden_act != "silu":
        raise ConfigError(f"failed to parse Qwen3 config: `hidden_act` {cfg.hidden_act!r} is not supported (silu)")
    if cfg.head_dim > 256:
        raise ConfigError(f"failed to parse Qwen3 config: `head_dim` {cfg.head_dim} is more than the 256 the kernels take")
    h, hd = cfg.hidden_size, cfg.head_dim
    layers = []
    for i in range(cfg.num_hidden_layers):
        p = f"model.layers.{i}."
        a = p + "self_attn."
        attn_w = {f"{x}_proj.weight": f"{a}{x}_proj.weight" for x in "qkvo"}
        if cfg.attention_bias:
            attn_w.update({f"{x}_proj.bias": f"{a}{x}_proj.bias" for x in "qkvo"})
        attn_w.update({"q_norm.weight": a + "q_norm.weight", "k_norm.weight": a + "k_norm.weight"})
        mixer = PartSpec("gqa_attention", dict(
            hidden_size=h, num_heads=cfg.num_attention_heads, num_kv_heads=cfg.num_key_value_heads, head_dim=hd,
            norm_eps=cfg.rms_norm_eps, qk_norm=True, bias=cfg.attention_bias, window=cfg.layer_window(i) or 0,
            position="rope"), attn_w)
        ffn = PartSpec("gated_mlp", dict(hidden_size=h, intermediate_size=cfg.intermediate_size,
                                         activation=cfg.hidden_act),
                       {f"{x}_proj.weight": f"{p}mlp.{x}_proj.weight" for x in ("gate", "up", "down")})
        norm = lambda name: PartSpec("rms_norm", dict(size=h, eps=cfg.rms_norm_eps), {"weight": p + name + ".weight"})
        layers.append(LayerSpec("prenorm", {"input_norm": norm("input_layernorm"), "mixer": mixer,
                                            "post_mixer_norm": norm("post_attention_layernorm"), "ffn": ffn}))
    embed_name = "model.embed_tokens.weight"
    return ModelSpec(
        architecture="Qwen3ForCausalLM", vocab_size=cfg.vocab_size, hidden_size=h,
        max_positions=cfg.max_position_embeddings, eos_token_ids=cfg.eos_token_ids,
        embedding=PartSpec("token_embedding", dict(vocab_size=cfg.vocab_size, hidden_size=h), {"weight": embed_name}),
        layers=layers, order=[RunSpec(i) for i in range(cfg.num_hidden_layers)],
        final_norm=PartSpec("rms_norm", dict(size=h, eps=cfg.rms_norm_eps), {"weight": "model.norm.weight"}),
        head=PartSpec("linear_head", dict(vocab_size=cfg.vocab_size, hidden_size=h),
                      {"weight": embed_name if cfg.tie_word_embeddings else "lm_head.weight"}),
        positions={"rope": PartSpec("rope", dict(rotary_dim=hd, max_positions=cfg.max_position_embeddings,
                                                 theta=cfg.rope_theta))},
        # a tied checkpoint may still carry the head it does not use (the reference never reads it,
        # crates/prelude-core/src/models/qwen3.rs:637-643), and old exports the rotary frequencies as a buffer
        ignored_tensors=("*.rotary_emb.inv_freq",) + (("lm_head.weight",) if cfg.tie_word_embeddings else ()))


QWEN3 = register_architecture(Architecture(
    name="qwen3", architecture_aliases=("Qwen3", "Qwen3Model"), model_type_aliases=("qwen3",),
    parse_config=Qwen3Config.from_dict, build_spec=qwen3_spec))
