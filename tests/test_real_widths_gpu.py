"""The engine at the layer widths of a real model (Qwen3-4B: hidden 2560, 32 heads over 8 KV heads of 128,
intermediate 9728) against the plain implementation.  Two layers and a vocabulary of 70,001 keep it small; the
tiny configurations never reach the kernels' wide variants (products over hundreds of tiles, the head over
thousands, vector norms, the decode attention that takes the raw projection), this does."""
import functools
import json
import os
import tempfile

import numpy as np
import pytest
import torch

import plain_model as pm
from helpers import check

pytestmark = pytest.mark.gpu
_keep = []


def wide_config() -> dict:
    return dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=70001, hidden_size=2560,
                intermediate_size=9728, num_hidden_layers=2, num_attention_heads=32, num_key_value_heads=8,
                head_dim=128, attention_bias=False, max_position_embeddings=1024, sliding_window=None,
                max_window_layers=2, tie_word_embeddings=True, rope_theta=1000000.0, rms_norm_eps=1e-6,
                use_sliding_window=False, hidden_act="silu", eos_token_id=70000)


@functools.lru_cache(maxsize=None)
def wide_model():
    """(folder, tokens, float64 logits of the plain implementation, its weights); weights stored in bfloat16 so that both
    paths of the engine and the plain implementation start from the same numbers."""
    from prelude_amd.weights import write_safetensors
    cfg = wide_config()
    w = pm.random_weights(cfg, seed=4, std=0.02, norm_std=0.02)
    w = {k: v.to(torch.bfloat16) for k, v in w.items()}
    tmp = tempfile.TemporaryDirectory(prefix="prelude_amd_test_wide_")
    _keep.append(tmp)
    with open(os.path.join(tmp.name, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_safetensors(os.path.join(tmp.name, "model.safetensors"), w)
    toks = torch.randint(0, cfg["vocab_size"], (96,), generator=torch.Generator().manual_seed(21)).tolist()
    w64 = {k: v.double() for k, v in w.items()}
    return tmp.name, toks, pm.forward(cfg, w64, toks), w64


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_whole_then_decoded_then_mixed(gpu, dtype):
    from prelude_amd.trace import TraceRunner
    folder, toks, ref, _ = wide_model()
    r = TraceRunner(folder, dtype, 512, page_size=16)
    n = len(toks)
    got = r.step([{"id": "whole", "tokens": toks, "want": list(range(n))}], ["whole"])
    check(got, ref, dtype, "whole")
    # most of it in one step, the last 32 one by one
    outs = [r.step([{"id": "d", "tokens": toks[:n - 32], "want": list(range(n - 32))}])]
    for i in range(n - 32, n):
        outs.append(r.step([{"id": "d", "tokens": [toks[i]], "want": [0]}]))
    r.step([], ["d"])
    check(np.concatenate(outs), ref, dtype, "decoded")
    # three requests a step: two decode (at different places) beside portions of a third
    for rid, upto in (("x", 40), ("y", 70)):
        r.step([{"id": rid, "tokens": toks[:upto], "want": []}])
    at = {"x": 40, "y": 70, "z": 0}
    rows = {k: [] for k in at}
    for size in (17, 2, 23, 5, 1, 9):
        entries = []
        for rid in ("x", "y"):
            entries.append({"id": rid, "tokens": [toks[at[rid]]], "want": [0]})
        entries.append({"id": "z", "tokens": toks[at["z"]:at["z"] + size], "want": list(range(size))})
        out = r.step(entries)
        rows["x"].append(out[0:1]), rows["y"].append(out[1:2]), rows["z"].append(out[2:])
        at["x"] += 1
        at["y"] += 1
        at["z"] += size
    check(np.concatenate(rows["x"]), ref[40:46], dtype, "mixed, first decoding request")
    check(np.concatenate(rows["y"]), ref[70:76], dtype, "mixed, second decoding request")
    check(np.concatenate(rows["z"]), ref[:57], dtype, "mixed, portions")
    r.step([], ["x", "y", "z"])
    assert r.engine.tables.audit() == "" and r.engine.tables.num_requests() == 0


def test_twenty_requests_decode_together(gpu):
    """Twenty requests at different places of the same sequence feed one token each, step after step: the decode
    attention that takes the raw projection (QK-norm, rotation and the cache write inside it) with more sequences
    than the products of few rows take, so the streaming and the library products feed it in turn."""
    from prelude_amd.trace import TraceRunner
    folder, toks, ref, _ = wide_model()
    r = TraceRunner(folder, "bfloat16", 20 * 96, page_size=16)
    starts = [3 + 4 * i for i in range(20)]
    for i, s in enumerate(starts):
        r.step([{"id": f"r{i}", "tokens": toks[:s], "want": []}])
    rows = [[] for _ in starts]
    for k in range(5):
        out = r.step([{"id": f"r{i}", "tokens": [toks[s + k]], "want": [0]} for i, s in enumerate(starts)])
        for i in range(len(starts)):
            rows[i].append(out[i:i + 1])
    for i, s in enumerate(starts):
        check(np.concatenate(rows[i]), ref[s:s + 5], "bfloat16", f"request {i} from position {s}")
    r.step([], [f"r{i}" for i in range(20)])
    assert r.engine.tables.audit() == "" and r.engine.tables.num_requests() == 0


def test_the_norm_inside_the_gated_product(gpu, monkeypatch):
    """Up to 16 rows at these widths the residual add and the norm behind the attention run inside the gated product:
    eight requests decode together with it and without it, both against the plain implementation, and the
    kernel is seen to run in the one case and not in the other."""
    from prelude_amd.ops import kernels as K
    from prelude_amd.trace import TraceRunner
    folder, toks, ref, _ = wide_model()
    calls = []
    inner = K.linear_gated_after_norm
    monkeypatch.setattr(K, "linear_gated_after_norm", lambda *a, **kw: (calls.append(a[0].shape[0]), inner(*a, **kw))[1])
    starts = [5 + 9 * i for i in range(8)]
    try:
        for on in (True, False):
            K.set_normed_gated(on)
            calls.clear()
            r = TraceRunner(folder, "bfloat16", 8 * 96, page_size=16)
            for i, s in enumerate(starts):
                r.step([{"id": f"r{i}", "tokens": toks[:s], "want": []}])
            seen = len(calls)
            rows = [[] for _ in starts]
            for k in range(4):
                out = r.step([{"id": f"r{i}", "tokens": [toks[s + k]], "want": [0]} for i, s in enumerate(starts)])
                for i in range(len(starts)):
                    rows[i].append(out[i:i + 1])
            for i, s in enumerate(starts):
                check(np.concatenate(rows[i]), ref[s:s + 4], "bfloat16", f"norm inside the product {on}, request {i}")
            # (a step replayed from a graph does not come by here again: at least the step that was recorded did)
            assert (set(calls[seen:]) == {8} and len(calls) - seen >= wide_config()["num_hidden_layers"]) if on else not calls, calls
            r.step([], [f"r{i}" for i in range(8)])
    finally:
        K.set_normed_gated(True)


@functools.lru_cache(maxsize=None)
def narrow_model():
    """The widths of a small model (Qwen3-0.6B: hidden 1,024, 16 heads over 8 KV heads of 128, intermediate 3,072), three
    layers, a small vocabulary: its o and down products have 64 tiles of 16 rows, which the streaming kernel cuts
    into slices of K for the norm behind them."""
    from prelude_amd.weights import write_safetensors
    cfg = dict(wide_config(), vocab_size=4099, eos_token_id=4098, hidden_size=1024, intermediate_size=3072,
               num_attention_heads=16, num_key_value_heads=8, num_hidden_layers=3, max_window_layers=3)
    w = pm.random_weights(cfg, seed=12, std=0.03, norm_std=0.02)
    w = {k: v.to(torch.bfloat16) for k, v in w.items()}
    tmp = tempfile.TemporaryDirectory(prefix="prelude_amd_test_narrow_")
    _keep.append(tmp)
    with open(os.path.join(tmp.name, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_safetensors(os.path.join(tmp.name, "model.safetensors"), w)
    toks = torch.randint(0, cfg["vocab_size"], (80,), generator=torch.Generator().manual_seed(5)).tolist()
    return tmp.name, toks, pm.forward(cfg, {k: v.double() for k, v in w.items()}, toks)


def test_narrow_widths_decode_with_their_products_in_slices(gpu, monkeypatch):
    """One request decoded token by token and nine decoding together at a small model's widths, where the last
    product of the attention and of the feed-forward come as slices of K from the streaming kernel: against the
    plain implementation, and the kernel is seen to run."""
    from prelude_amd.ops import kernels as K
    from prelude_amd.trace import TraceRunner
    folder, toks, ref = narrow_model()
    calls = []
    inner = K.gemm_skinny_sliced
    monkeypatch.setattr(K, "gemm_skinny_sliced", lambda *a, **kw: (calls.append(a[0].shape[0]), inner(*a, **kw))[1])
    r = TraceRunner(folder, "bfloat16", 10 * 96, page_size=16)
    n = len(toks)
    outs = [r.step([{"id": "d", "tokens": toks[:n - 24], "want": list(range(n - 24))}])]
    for i in range(n - 24, n):
        outs.append(r.step([{"id": "d", "tokens": [toks[i]], "want": [0]}]))
    r.step([], ["d"])
    check(np.concatenate(outs), ref, "bfloat16", "decoded")
    assert calls and set(calls) == {1}
    calls.clear()
    starts = [4 + 7 * i for i in range(9)]
    for i, s in enumerate(starts):
        r.step([{"id": f"r{i}", "tokens": toks[:s], "want": []}])
    rows = [[] for _ in starts]
    for k in range(4):
        out = r.step([{"id": f"r{i}", "tokens": [toks[s + k]], "want": [0]} for i, s in enumerate(starts)])
        for i in range(len(starts)):
            rows[i].append(out[i:i + 1])
    for i, s in enumerate(starts):
        check(np.concatenate(rows[i]), ref[s:s + 4], "bfloat16", f"request {i} from position {s}")
    assert 9 in calls
    r.step([], [f"r{i}" for i in range(9)])
    assert r.engine.tables.audit() == "" and r.engine.tables.num_requests() == 0


def test_graph_replays_equal_eager_steps_at_real_widths(gpu):
    """Decode steps of one, five and twelve requests at these widths (the streaming products, the gated product with
    the norm inside it, the decode attention on the raw projection) replayed from graphs give the bits of the same
    steps run directly, with prompt portions between the replays."""
    from prelude_amd.config import EngineConfig
    from prelude_amd.engine import Engine, StepEntry
    folder, toks, _, _ = wide_model()

    def play(hip_graph):
        eng = Engine.from_model_dir(folder, EngineConfig(dtype="bfloat16", page_size=16, max_cache_tokens=12 * 96,
                                                         hip_graph=hip_graph))
        outs, at = [], {}

        def feed(parts):
            entries = []
            for r, n in parts:
                lo = at.get(r, 0)
                entries.append(StepEntry(r, toks[lo:lo + n], [n - 1]))
                at[r] = lo + n
            outs.append(eng.step(entries).cpu())
        feed([(0, 30)])
        for _ in range(4):
            feed([(0, 1)])
        feed([(r, 10 + 3 * r) for r in range(1, 5)])
        for _ in range(4):
            feed([(r, 1) for r in range(5)])
        feed([(r, 5 + r) for r in range(5, 12)])
        for _ in range(4):
            feed([(r, 1) for r in range(12)])
        for _ in range(2):
            feed([(0, 1)])
        return eng, outs

    eager_eng, eager = play(False)
    graph_eng, graphed = play(True)
    assert eager_eng._graphs is None and graph_eng._graphs.captures == 3 and graph_eng._graphs.replays >= 11
    for i, (a, b) in enumerate(zip(eager, graphed)):
        assert torch.equal(a, b), f"step {i}: the replay differs from the eager step"


@pytest.mark.parametrize("batch", [33, 64, 100, 128])
def test_many_requests_decode_together(gpu, batch):
    """Decode steps of 33 to 128 requests at the real widths: the products of 17 to 128 rows (X through LDS, the
    narrow ones in slices of K that the norm adds, the gated one with its activation in the epilogue), the head at
    up to 64 rows through the same kernel and beyond through the library, the decode attention over that many
    sequences; up to 64 requests are replayed from a graph after the first step, more are launched directly."""
    from prelude_amd.trace import TraceRunner
    folder, toks, ref, _ = wide_model()
    r = TraceRunner(folder, "bfloat16", batch * 112, page_size=16)
    starts = [2 + (7 * i) % 88 for i in range(batch)]
    for i, s in enumerate(starts):
        r.step([{"id": f"r{i}", "tokens": toks[:s], "want": []}])
    rows = [[] for _ in starts]
    steps = 4
    for k in range(steps):
        out = r.step([{"id": f"r{i}", "tokens": [toks[s + k]], "want": [0]} for i, s in enumerate(starts)])
        for i in range(batch):
            rows[i].append(out[i:i + 1])
    for i, s in enumerate(starts):
        check(np.concatenate(rows[i]), ref[s:s + steps], "bfloat16", f"request {i} of {batch} from position {s}")
    r.step([], [f"r{i}" for i in range(batch)])
    assert r.engine.tables.audit() == "" and r.engine.tables.num_requests() == 0


def test_greedy_generation_at_real_widths(gpu):
    from prelude_amd import LLM
    folder, toks, _, w64 = wide_model()
    llm = LLM(folder, dtype="float32", max_cache_tokens=512)
    res = llm.generate([toks[:20]], max_tokens=4, temperature=0.0)[0]
    assert res.token_ids == pm.greedy(wide_config(), w64, toks[:20], 4)


@functools.lru_cache(maxsize=None)
def long_model():
    """The same layer widths under a small vocabulary, for a sequence of 700 tokens.  With these weights a split
    of 256 keys that is left out of one layer's attention moves the logits of the positions behind it by 0.34 to
    0.92 of their spread (second layer) or 2.7 to 4.7 (first layer), measured with the plain implementation; the
    bound for bfloat16 is a tenth of the spread and the engine's error 0.06 of it."""
    from prelude_amd.weights import write_safetensors
    cfg = dict(wide_config(), vocab_size=4099, eos_token_id=4098)
    w = pm.random_weights(cfg, seed=9, std=0.02, norm_std=0.02)
    w = {k: v.to(torch.bfloat16) for k, v in w.items()}
    tmp = tempfile.TemporaryDirectory(prefix="prelude_amd_test_long_")
    _keep.append(tmp)
    with open(os.path.join(tmp.name, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_safetensors(os.path.join(tmp.name, "model.safetensors"), w)
    toks = torch.randint(0, cfg["vocab_size"], (700,), generator=torch.Generator().manual_seed(33)).tolist()
    return tmp.name, toks, pm.forward(cfg, {k: v.double() for k, v in w.items()}, toks)


def test_decoding_far_into_a_context_from_graphs(gpu):
    """What serving runs at this width -- the decode attention that takes the raw projection, over several splits
    of 256 keys with their merge, replayed from a captured graph -- against the plain implementation: 560 tokens
    in one step and the next 32 one by one, then three requests decoding together while their contexts pass 256
    and 512 keys (one split becomes two, two become three)."""
    from prelude_amd.trace import TraceRunner
    folder, toks, ref = long_model()
    r = TraceRunner(folder, "bfloat16", 2048, page_size=16)
    assert r.engine._graphs is not None
    outs = [r.step([{"id": "d", "tokens": toks[:560], "want": [0, 255, 256, 559]}])]
    check(outs[0], ref[[0, 255, 256, 559]], "bfloat16", "the portion")
    rows = [r.step([{"id": "d", "tokens": [toks[i]], "want": [0]}]) for i in range(560, 592)]
    check(np.concatenate(rows), ref[560:592], "bfloat16", "decoded from position 560")
    replays = r.engine._graphs.replays
    assert replays == 32 and r.engine._graphs.captures == 1
    r.step([], ["d"])
    starts = {"x": 250, "y": 505, "z": 660}
    for rid, s0 in starts.items():
        r.step([{"id": rid, "tokens": toks[:s0], "want": []}])
    got = {rid: [] for rid in starts}
    for k in range(14):
        out = r.step([{"id": rid, "tokens": [toks[s0 + k]], "want": [0]} for rid, s0 in starts.items()])
        for j, rid in enumerate(starts):
            got[rid].append(out[j:j + 1])
    assert r.engine._graphs.replays == replays + 14
    for rid, s0 in starts.items():
        check(np.concatenate(got[rid]), ref[s0:s0 + 14], "bfloat16", f"request decoding from position {s0}")
    r.step([], list(starts))
    assert r.engine.tables.audit() == "" and r.engine.tables.num_requests() == 0


@functools.lru_cache(maxsize=None)
def context_model():
    """The same widths and small vocabulary for a sequence of 4,100 tokens; the plain implementation in 32-bit (six
    seconds on the CPU).  Measured with the plain implementation: a split of 256 keys left out of the first
    layer's attention moves the last positions' logits by 0.9 to 1.3 of their spread wherever the split lies, one
    left out of the second layer's by 0.05 to 0.15; the plain implementation with every operation rounded to
    bfloat16 is off by 0.07, and the bound is a tenth of the spread."""
    from prelude_amd.weights import write_safetensors
    cfg = dict(wide_config(), vocab_size=4099, eos_token_id=4098, max_position_embeddings=4352)
    w = pm.random_weights(cfg, seed=9, std=0.02, norm_std=0.02)
    w = {k: v.to(torch.bfloat16) for k, v in w.items()}
    tmp = tempfile.TemporaryDirectory(prefix="prelude_amd_test_context_")
    _keep.append(tmp)
    with open(os.path.join(tmp.name, "config.json"), "w") as f:
        json.dump(cfg, f)
    write_safetensors(os.path.join(tmp.name, "model.safetensors"), w)
    toks = torch.randint(0, cfg["vocab_size"], (4100,), generator=torch.Generator().manual_seed(33)).tolist()
    return tmp.name, toks, pm.forward(cfg, {k: v.float() for k, v in w.items()}, toks, dtype=torch.float32).double()


def test_eight_requests_decode_at_4096_tokens_from_graphs(gpu):
    """The step the benchmark times, against the plain implementation: eight requests with some 4,000 tokens behind
    them feed one token each, twelve steps, replayed from one captured graph.  Eight KV heads x 16 splits x 8
    sequences are 1,024 workgroups: the decode attention that takes the raw projection in its two-wavefront form,
    with the merge of 16 splits.  One request starts on a split's edge (3,840 = 15 x 256), one a token behind it,
    one on a page's edge (4,000), and the last ends at 4,096 exactly."""
    from prelude_amd.trace import TraceRunner
    folder, toks, ref = context_model()
    starts = [3840, 3841, 3900, 4000, 4032, 4070, 4080, 4084]
    steps = 12
    r = TraceRunner(folder, "bfloat16", len(starts) * 4160, page_size=16)
    assert r.engine._graphs is not None
    for i, s0 in enumerate(starts):
        for lo in range(0, s0, 2048):
            r.step([{"id": i, "tokens": toks[lo:min(s0, lo + 2048)], "want": []}])
    rows = [[] for _ in starts]
    for k in range(steps):
        out = r.step([{"id": i, "tokens": [toks[s0 + k]], "want": [0]} for i, s0 in enumerate(starts)])
        for i in range(len(starts)):
            rows[i].append(out[i:i + 1])
    assert r.engine._graphs.replays == steps and r.engine._graphs.captures == 1
    for i, s0 in enumerate(starts):
        check(np.concatenate(rows[i]), ref[s0:s0 + steps], "bfloat16", f"request decoding from position {s0}")
    r.step([], list(range(len(starts))))
    assert r.engine.tables.audit() == "" and r.engine.tables.num_requests() == 0
