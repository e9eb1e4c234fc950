"""Typed model configuration read from an architecture's own config.json keys.

The keys, which of them are required, and the error for a missing one follow
crates/prelude-core/src/models/config.rs:4-22 (every field required except
``sliding_window``) and crates/prelude-core/src/engine/config.rs:122-170
(``eos_token_id``: an integer or a non-empty list, required for generation).
"""
from __future__ import annotations

import dataclasses
import json
import os
from typing import Any, Mapping, Optional, Tuple


class ConfigError(ValueError):
    """A config.json that cannot be used; the message names the key."""


_MISSING = object()


def _get(raw: Mapping[str, Any], key: str, kind, arch: str, default=_MISSING):
    if key not in raw or raw[key] is None:
        if default is not _MISSING:
            return default
        raise ConfigError(f"failed to parse {arch} config: missing required key `{key}`")
    v = raw[key]
    if kind is bool:
        if not isinstance(v, bool):
            raise ConfigError(f"failed to parse {arch} config: `{key}` must be true or false, got {v!r}")
        return v
    if kind is int:
        if isinstance(v, bool) or not isinstance(v, int):
            raise ConfigError(f"failed to parse {arch} config: `{key}` must be an integer, got {v!r}")
        if v < 0:
            raise ConfigError(f"failed to parse {arch} config: `{key}` must not be negative, got {v!r}")
        return v
    if kind is float:
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"failed to parse {arch} config: `{key}` must be a number, got {v!r}")
        return float(v)
    if kind is str:
        if not isinstance(v, str):
            raise ConfigError(f"failed to parse {arch} config: `{key}` must be a string, got {v!r}")
        return v
    raise AssertionError(kind)


def parse_eos_token_ids(raw: Mapping[str, Any]) -> Tuple[int, ...]:
    """``eos_token_id`` as a tuple (crates/prelude-core/src/engine/config.rs:122-170)."""
    if "eos_token_id" not in raw or raw["eos_token_id"] is None:
        raise ConfigError("generation model config is missing required field `eos_token_id`")
    v = raw["eos_token_id"]
    if isinstance(v, bool):
        raise ConfigError("generation model config has invalid `eos_token_id` type")
    if isinstance(v, int):
        if v < 0:
            raise ConfigError("generation model config has invalid non-integer `eos_token_id`")
        return (v,)
    if isinstance(v, list):
        if not v:
            raise ConfigError("generation model config has empty `eos_token_id`")
        for e in v:
            if isinstance(e, bool) or not isinstance(e, int) or e < 0:
                raise ConfigError("generation model config has non-integer entry in `eos_token_id`")
        return tuple(v)
    raise ConfigError("generation model config has invalid `eos_token_id` type")


@dataclasses.dataclass(frozen=True)
class Qwen3Config:
    """Qwen3 dense (crates/prelude-core/src/models/config.rs:4-22)."""

    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    attention_bias: bool
    max_position_embeddings: int
    sliding_window: Optional[int]
    max_window_layers: int
    tie_word_embeddings: bool
    rope_theta: float
    rms_norm_eps: float
    use_sliding_window: bool
    hidden_act: str
    eos_token_ids: Tuple[int, ...]

    ARCH = "Qwen3"

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "Qwen3Config":
        a = cls.ARCH
        cfg = cls(
            vocab_size=_get(raw, "vocab_size", int, a),
            hidden_size=_get(raw, "hidden_size", int, a),
            intermediate_size=_get(raw, "intermediate_size", int, a),
            num_hidden_layers=_get(raw, "num_hidden_layers", int, a),
            num_attention_heads=_get(raw, "num_attention_heads", int, a),
            num_key_value_heads=_get(raw, "num_key_value_heads", int, a),
            head_dim=_get(raw, "head_dim", int, a),
            attention_bias=_get(raw, "attention_bias", bool, a),
            max_position_embeddings=_get(raw, "max_position_embeddings", int, a),
            sliding_window=_get(raw, "sliding_window", int, a, default=None),
            max_window_layers=_get(raw, "max_window_layers", int, a),
            tie_word_embeddings=_get(raw, "tie_word_embeddings", bool, a),
            rope_theta=_get(raw, "rope_theta", float, a),
            rms_norm_eps=_get(raw, "rms_norm_eps", float, a),
            use_sliding_window=_get(raw, "use_sliding_window", bool, a),
            hidden_act=_get(raw, "hidden_act", str, a),
            eos_token_ids=parse_eos_token_ids(raw),
        )
        cfg.validate()
        return cfg

    def validate(self) -> None:
        a = self.ARCH
        for key in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                    "num_attention_heads", "num_key_value_heads", "head_dim", "max_position_embeddings"):
            if getattr(self, key) <= 0:
                raise ConfigError(f"failed to parse {a} config: `{key}` must be positive")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(
                f"failed to parse {a} config: `num_attention_heads` ({self.num_attention_heads}) is not a "
                f"multiple of `num_key_value_heads` ({self.num_key_value_heads})")
        if self.head_dim % 2:
            raise ConfigError(f"failed to parse {a} config: `head_dim` ({self.head_dim}) must be even for RoPE")
        if self.rms_norm_eps <= 0 or self.rope_theta <= 0:
            raise ConfigError(f"failed to parse {a} config: `rms_norm_eps` and `rope_theta` must be positive")
        if self.use_sliding_window and not self.sliding_window:
            raise ConfigError(f"failed to parse {a} config: `use_sliding_window` is true but `sliding_window` is unset")
        for e in self.eos_token_ids:
            if e >= self.vocab_size:
                raise ConfigError(f"failed to parse {a} config: `eos_token_id` {e} is outside the vocabulary")

    def layer_window(self, layer: int) -> Optional[int]:
        """Keys a layer attends to, or None for all of them.

        The reference parses the three window keys and refuses
        ``use_sliding_window`` (crates/prelude-core/src/models/qwen3.rs:50-52).
        Here they mean: layers with index >= ``max_window_layers`` see the
        last ``sliding_window`` keys, the query's own included.
        """
        if self.use_sliding_window and self.sliding_window and layer >= self.max_window_layers:
            return int(self.sliding_window)
        return None

    def to_dict(self) -> dict:
        d = dataclasses.asdict(self)
        eos = d.pop("eos_token_ids")
        d["eos_token_id"] = eos[0] if len(eos) == 1 else list(eos)
        d["architectures"] = ["Qwen3ForCausalLM"]
        d["model_type"] = "qwen3"
        return d


def read_config_json(model_dir: str) -> dict:
    path = os.path.join(model_dir, "config.json")
    try:
        with open(path, "r", encoding="utf-8") as f:
            raw = json.load(f)
    except FileNotFoundError:
        raise ConfigError(f"no config.json in model folder {model_dir!r}") from None
    except json.JSONDecodeError as e:
        raise ConfigError(f"failed to parse {path}: {e}") from None
    if not isinstance(raw, dict):
        raise ConfigError(f"failed to parse {path}: top level is not an object")
    return raw
