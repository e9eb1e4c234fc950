"""Configuration and registry (no GPU)."""
import json

import pytest

import plain_model as pm
from prelude_amd import models  # noqa: F401  registers Qwen3
from prelude_amd.config import (ConfigError, Qwen3Config, UnknownArchitecture, read_config_json,
                                registered_architectures, resolve_architecture)
from prelude_amd.models.qwen3 import qwen3_spec


def test_parse_all_keys():
    raw = pm.tiny_config_b()
    cfg = Qwen3Config.from_dict(raw)
    assert (cfg.vocab_size, cfg.hidden_size, cfg.intermediate_size, cfg.num_hidden_layers) == (509, 96, 160, 3)
    assert (cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim) == (6, 1, 32)
    assert cfg.rope_theta == 1e6 and cfg.rms_norm_eps == 1e-5 and cfg.max_position_embeddings == 256
    assert cfg.tie_word_embeddings is False and cfg.eos_token_ids == (507, 508)
    assert cfg.sliding_window is None and cfg.layer_window(2) is None
    assert Qwen3Config.from_dict(cfg.to_dict()) == cfg


@pytest.mark.parametrize("key", ["vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                                 "num_attention_heads", "num_key_value_heads", "head_dim", "attention_bias",
                                 "max_position_embeddings", "max_window_layers", "tie_word_embeddings", "rope_theta",
                                 "rms_norm_eps", "use_sliding_window", "hidden_act", "eos_token_id"])
def test_every_key_is_required(key):
    # crates/prelude-core/src/models/config.rs:4-22: no defaults except sliding_window
    raw = pm.tiny_config_a()
    del raw[key]
    with pytest.raises(ConfigError, match=key):
        Qwen3Config.from_dict(raw)


def test_sliding_window_is_optional_and_types_are_checked():
    raw = pm.tiny_config_a()
    del raw["sliding_window"]
    assert Qwen3Config.from_dict(raw).sliding_window is None
    for key, bad in (("vocab_size", "256"), ("attention_bias", 0), ("rope_theta", "1e4"), ("hidden_size", 64.5),
                     ("eos_token_id", []), ("eos_token_id", "2"), ("eos_token_id", [1, 2.5])):
        with pytest.raises(ConfigError):
            Qwen3Config.from_dict(dict(pm.tiny_config_a(), **{key: bad}))
    with pytest.raises(ConfigError, match="multiple"):
        Qwen3Config.from_dict(dict(pm.tiny_config_a(), num_attention_heads=5))
    with pytest.raises(ConfigError, match="eos"):
        Qwen3Config.from_dict(dict(pm.tiny_config_a(), eos_token_id=256))


def test_window_layers():
    cfg = Qwen3Config.from_dict(pm.tiny_config_c())
    assert [cfg.layer_window(i) for i in range(4)] == [None, None, 24, 24]
    assert [pm.layer_window(pm.tiny_config_c(), i) for i in range(4)] == [None, None, 24, 24]
    with pytest.raises(ConfigError, match="sliding_window"):
        Qwen3Config.from_dict(dict(pm.tiny_config_c(), sliding_window=None))


def test_registry_resolution():
    # crates/prelude-core/src/models/registry.rs:198-296
    assert "qwen3" in registered_architectures()
    assert resolve_architecture({"architectures": ["Qwen3ForCausalLM"]}).name == "qwen3"
    assert resolve_architecture({"architectures": ["qwen_3ForCausalLM"]}).name == "qwen3"       # normalisation
    assert resolve_architecture({"architectures": ["Other"], "model_type": "qwen3"}).name == "qwen3"
    assert resolve_architecture({"model_type": "Qwen3"}).name == "qwen3"
    for raw in ({"architectures": ["LlamaForCausalLM"]}, {"architectures": ["Qwen3ForSequenceClassification"]}, {},
                {"model_type": "gpt2"}):
        with pytest.raises(UnknownArchitecture, match="unable to resolve"):
            resolve_architecture(raw)


def test_spec_is_data_from_the_config():
    cfg = Qwen3Config.from_dict(pm.tiny_config_c())
    spec = qwen3_spec(cfg)
    assert len(spec.layers) == 4 and [r.layer for r in spec.order] == [0, 1, 2, 3]
    m = spec.layers[3].parts["mixer"]
    assert m.kind == "gqa_attention" and m.params["window"] == 24 and m.params["bias"] is True
    assert m.params["head_dim"] == 48 and m.params["num_kv_heads"] == 2 and m.params["norm_eps"] == 3e-6
    assert spec.layers[0].parts["mixer"].params["window"] == 0
    assert spec.layers[1].parts["ffn"].params["intermediate_size"] == 112
    assert spec.positions["rope"].params == dict(rotary_dim=48, max_positions=512, theta=50000.0)
    assert spec.head.weights["weight"] == "lm_head.weight"
    tied = qwen3_spec(Qwen3Config.from_dict(pm.tiny_config_a()))
    assert tied.head.weights["weight"] == tied.embedding.weights["weight"] == "model.embed_tokens.weight"
    with pytest.raises(ConfigError, match="head_dim"):
        qwen3_spec(Qwen3Config.from_dict(dict(pm.tiny_config_a(), head_dim=258)))
    assert qwen3_spec(Qwen3Config.from_dict(dict(pm.tiny_config_a(), head_dim=24))).layers[0].parts["mixer"].params["head_dim"] == 24
    with pytest.raises(ConfigError, match="hidden_act"):
        qwen3_spec(Qwen3Config.from_dict(dict(pm.tiny_config_a(), hidden_act="gelu")))


def test_read_config_json(tmp_path):
    with pytest.raises(ConfigError, match="config.json"):
        read_config_json(str(tmp_path))
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="parse"):
        read_config_json(str(tmp_path))
    (tmp_path / "config.json").write_text(json.dumps(pm.tiny_config_a()))
    assert read_config_json(str(tmp_path))["hidden_size"] == 64


def test_where_a_step_with_portions_is_worth_a_graph():
    """Steps with prompt portions are replayed from graphs up to the number of tokens at which the device's work
    is taken to reach the host's launches: some hundreds for a small model, about 140 for a 36-layer model of 4 G
    matrix elements, none where streaming the weights alone takes longer than the launches; never beyond the
    configured number, and the matrix elements are counted from the model's own tensors."""
    from prelude_amd.engine.graph import portion_tokens_worth_a_graph as worth
    assert 600 < worth(int(0.6e9), 28 * 9 + 3, 2, 1024) < 900
    assert worth(int(0.6e9), 28 * 9 + 3, 2, 256) == 256
    assert 100 < worth(int(4.0e9), 36 * 9 + 3, 2, 1024) < 200
    assert worth(int(8.2e9), 36 * 9 + 3, 2, 1024) == 0
    assert worth(int(0.6e9), 28 * 9 + 3, 2, 0) == 0
    from prelude_amd.models.causal_lm import CausalLM
    from prelude_amd.config import resolve_architecture
    for cfg in (pm.tiny_config_a(), pm.tiny_config_b(), pm.tiny_config_c()):
        arch = resolve_architecture(cfg)
        model = CausalLM(arch.build_spec(arch.parse_config(cfg)))
        shapes = pm.tensor_shapes(cfg)
        want = sum(a * b for name, (a, *rest) in shapes.items() for b in rest
                   if name != "model.embed_tokens.weight" or cfg["tie_word_embeddings"])
        assert model.matrix_elements() == want and model.graph_safe_portions
        # the launches are the parts' own counts: two norms, a mixer of four and a feed-forward of three a layer
        assert model.launches_per_step() == 9 * cfg["num_hidden_layers"] + 3
