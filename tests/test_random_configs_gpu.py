"""Configurations drawn at random (fixed seeds): every size and option that config.json allows should either run
and agree with the plain implementation or be refused with an error that says why -- never give a wrong result.
Each drawn model is replayed whole, in portions beside a decoding request, and token by token, in 32-bit and in
bfloat16."""
import json
import os
import tempfile

import numpy as np
import pytest
import torch

import plain_model as pm
from helpers import check

pytestmark = pytest.mark.gpu


def draw_config(seed: int) -> tuple:
    rng = np.random.default_rng(seed)
    hd = int(rng.choice([16, 32, 48, 64, 80, 96, 112, 128, 256]))
    nkv = int(rng.choice([1, 2, 3, 4]))
    group = int(rng.choice([1, 2, 3, 4, 5, 8]))
    layers = int(rng.integers(1, 4))
    window = int(rng.choice([0, 0, 5, 16, 33]))
    cfg = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3",
               vocab_size=int(rng.integers(50, 700)), hidden_size=int(rng.choice([24, 40, 72, 100, 136, 200])),
               intermediate_size=int(rng.choice([16, 56, 88, 130, 250])), num_hidden_layers=layers,
               num_attention_heads=nkv * group, num_key_value_heads=nkv, head_dim=hd,
               attention_bias=bool(rng.integers(0, 2)), max_position_embeddings=256,
               sliding_window=window or None, max_window_layers=int(rng.integers(0, layers + 1)),
               tie_word_embeddings=bool(rng.integers(0, 2)), rope_theta=float(rng.choice([100.0, 10000.0, 1e6])),
               rms_norm_eps=float(rng.choice([1e-6, 1e-5, 3e-4])), use_sliding_window=bool(window),
               hidden_act="silu", eos_token_id=0)
    page = int(rng.choice([4, 8, 16, 32, 64, 128]))
    return cfg, page


@pytest.mark.parametrize("seed", list(range(int(os.environ.get("PRELUDE_AMD_DRAWN_CONFIGS", "12")))))   # widen for a hunt
def test_drawn_configuration(gpu, seed):
    from prelude_amd.trace import TraceRunner
    from prelude_amd.weights import write_safetensors
    cfg, page = draw_config(seed)
    w = pm.random_weights(cfg, seed=100 + seed, std=0.08, norm_std=0.05)
    rng = np.random.default_rng(1000 + seed)
    toks = rng.integers(0, cfg["vocab_size"], size=90).tolist()
    # the bfloat16 engine rounds the weights it loads: the plain model gets the same rounded weights, so that what
    # is compared is the engine's arithmetic and not the rounding of the file's values
    refs = {"float32": pm.forward(cfg, w, toks),
            "bfloat16": pm.forward(cfg, {k: v.to(torch.bfloat16).float() for k, v in w.items()}, toks)}
    with tempfile.TemporaryDirectory(prefix="prelude_amd_drawn_") as folder:
        with open(os.path.join(folder, "config.json"), "w") as f:
            json.dump(cfg, f)
        write_safetensors(os.path.join(folder, "model.safetensors"), w)
        for dtype in ("float32", "bfloat16"):
            ref = refs[dtype]
            what = f"seed {seed} {dtype} page {page} {cfg}"
            r = TraceRunner(folder, dtype, 512, page_size=page)
            got = r.step([{"id": "w", "tokens": toks, "want": list(range(90))}], ["w"])
            check(got, ref, dtype, "whole: " + what)
            # portions of one request beside another that decodes from position 50 on
            r.step([{"id": "d", "tokens": toks[:50], "want": []}])
            at, a, b = 0, [], []
            for k, n in enumerate((3, 29, 2, 17, 1, 38)):
                out = r.step([{"id": "p", "tokens": toks[at:at + n], "want": list(range(n))},
                              {"id": "d", "tokens": [toks[50 + k]], "want": [0]}])
                a.append(out[:n]), b.append(out[n:])
                at += n
            check(np.concatenate(a), ref, dtype, "portions: " + what)
            check(np.concatenate(b), ref[50:56], dtype, "decoding beside portions: " + what)
            # decode alone (the path of a step of single tokens)
            outs = [r.step([{"id": "d", "tokens": [toks[i]], "want": [0]}]) for i in range(56, 70)]
            check(np.concatenate(outs), ref[56:70], dtype, "decoding alone: " + what)
            r.step([], ["p", "d"])
            assert r.engine.tables.audit() == "" and r.engine.tables.num_requests() == 0


@pytest.mark.parametrize("hd,nh,nkv,hidden", [(8, 4, 2, 40), (20, 3, 1, 50), (24, 6, 2, 72), (40, 2, 2, 100), (250, 2, 1, 36)])
def test_head_sizes_outside_steps_of_16(gpu, hd, nh, nkv, hidden):
    """Head sizes that are no multiple of 16 (and widths that are no multiple of 8) are not refused: the generic
    kernels take them, in 32-bit and in bfloat16, whole and in portions beside a decoding request."""
    from prelude_amd.trace import TraceRunner
    from prelude_amd.weights import write_safetensors
    cfg = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=203, hidden_size=hidden,
               intermediate_size=60, num_hidden_layers=2, num_attention_heads=nh, num_key_value_heads=nkv, head_dim=hd,
               attention_bias=False, max_position_embeddings=128, sliding_window=None, max_window_layers=2,
               tie_word_embeddings=True, rope_theta=10000.0, rms_norm_eps=1e-6, use_sliding_window=False,
               hidden_act="silu", eos_token_id=0)
    w = pm.random_weights(cfg, seed=hd, std=0.08, norm_std=0.05)
    toks = np.random.default_rng(hd).integers(0, 203, size=70).tolist()
    refs = {"float32": pm.forward(cfg, w, toks),
            "bfloat16": pm.forward(cfg, {k: v.to(torch.bfloat16).float() for k, v in w.items()}, toks)}
    with tempfile.TemporaryDirectory(prefix="prelude_amd_hd_") as folder:
        with open(os.path.join(folder, "config.json"), "w") as f:
            json.dump(cfg, f)
        write_safetensors(os.path.join(folder, "model.safetensors"), w)
        for dtype in ("float32", "bfloat16"):
            r = TraceRunner(folder, dtype, 256, page_size=16)
            got = r.step([{"id": "w", "tokens": toks, "want": list(range(70))}], ["w"])
            check(got, refs[dtype], dtype, f"whole, head_dim {hd} {dtype}")
            r.step([{"id": "d", "tokens": toks[:40], "want": []}])
            at, a, b = 0, [], []
            for k, n in enumerate((19, 2, 30, 1, 18)):
                out = r.step([{"id": "p", "tokens": toks[at:at + n], "want": list(range(n))},
                              {"id": "d", "tokens": [toks[40 + k]], "want": [0]}])
                a.append(out[:n]), b.append(out[n:])
                at += n
            check(np.concatenate(a), refs[dtype], dtype, f"portions, head_dim {hd} {dtype}")
            check(np.concatenate(b), refs[dtype][40:45], dtype, f"decoding, head_dim {hd} {dtype}")
