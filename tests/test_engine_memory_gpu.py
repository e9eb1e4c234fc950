"""How the engine sizes what it allocates: the page pools from a measured step, a pool of its own size per cache
group, a bounded cache of captured decode steps."""
import numpy as np
import pytest
import torch

from helpers import check, model_folder, reference_logits

pytestmark = pytest.mark.gpu


def mid_config() -> dict:
    """Narrow layers under a full-size vocabulary: the logits are what a step's memory is made of."""
    return dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=151936, hidden_size=512,
                intermediate_size=1536, num_hidden_layers=2, num_attention_heads=8, num_key_value_heads=2,
                head_dim=64, attention_bias=False, max_position_embeddings=131072, sliding_window=None,
                max_window_layers=2, tie_word_embeddings=True, rope_theta=1000000.0, rms_norm_eps=1e-6,
                use_sliding_window=False, hidden_act="silu", eos_token_id=151645)


def test_pool_sized_from_a_measured_step(gpu):
    """``max_cache_tokens=None``: the pool is what the device has left after the weights, a measured step of
    ``max_num_batched_tokens`` tokens and the stated reserves.  Then the worst the engine is configured for is run
    -- a portion of 8,192 tokens, decode steps of 64 requests captured at several table widths, portions of 250
    and 256 tokens captured when their shape comes a second time -- and the device must still hold no more than
    the share it was given."""
    from prelude_amd.config import EngineConfig
    from prelude_amd.engine import Engine, StepEntry
    torch.cuda.empty_cache()
    total = torch.cuda.mem_get_info(gpu)[1]
    share = 0.03                                          # a small share keeps the test's pool small (some GB)
    cfg = EngineConfig(dtype="bfloat16", gpu_memory_utilization=share, max_num_batched_tokens=8192,
                       max_running_requests=64, hip_graph_max_bs=64, hip_graph_cache_size=4)
    eng = Engine.from_config(mid_config(), cfg, seed=1)
    plan = eng.memory_plan
    assert plan["step_peak"] > 512 * 151936 * 4          # the probe saw the logits of its wanted rows
    # a logits tensor per kept graph, the decode steps' activations, and a share of the measured step for the
    # captured steps with portions: this model's are worth a graph up to some 380 of the step's 8,192 tokens
    worth = eng._graphs.portion_tokens
    assert 256 <= worth < 512
    assert plan["graphs"] == 4 * 64 * 151936 * 4 + (256 << 20) + plan["step_peak"] * worth // 8192
    assert plan["cache"] > 0 and eng.cache_tokens >= 16 * 16
    per_token = 2 * 2 * 2 * 64 * 2
    assert abs(eng.cache_tokens * per_token - plan["cache"]) <= 32 * per_token      # the budget is what was allocated
    rng = np.random.default_rng(0)
    v = 151936
    # the longest step there is, wanting as many rows as the probe assumed
    eng.step([StepEntry(0, rng.integers(0, v, 8192).tolist(), list(range(8192 - 512, 8192)))])
    eng.release(0)
    # 64 decoding requests, captured at three table widths (contexts under 1,024, 2,048 and 3,072 tokens)
    for r in range(64):
        for _ in range(4):
            eng.step([StepEntry(100 + r, rng.integers(0, v, 250).tolist(), [])])
    for width in range(3):
        for _ in range(2):
            eng.step([StepEntry(100 + r, [int(rng.integers(0, v))], [0]) for r in range(64)])
        if width < 2:
            for r in range(64):
                for _ in range(4):
                    eng.step([StepEntry(100 + r, rng.integers(0, v, 256).tolist(), [])])
    # three shapes of decode steps and four of portions (250 tokens from the start; 250 behind as many or more; 256
    # behind 1,001 and behind 2,026, with wider tables), four kept at a time
    assert eng._graphs.captures == 7 and eng._graphs.evictions == 3
    torch.cuda.synchronize()
    free, _ = torch.cuda.mem_get_info(gpu)
    assert total - free <= share * total, f"{(total - free) >> 20} MB in use, the share was {int(share * total) >> 20} MB"
    for r in range(64):
        eng.release(100 + r)
    assert eng.tables.audit() == ""


def test_captured_steps_are_kept_up_to_a_number(gpu):
    """More shapes of decode steps than graphs are kept: the least recently used one goes and is captured again
    when its shape comes back, and every step gives what the eager step gives, bit for bit."""
    from prelude_amd.config import EngineConfig
    from prelude_amd.engine import Engine, StepEntry
    folder, cfg, _ = model_folder("b")
    seqs = [reference_logits("b", 40 + i, 120)[0] for i in range(4)]

    def play(hip_graph):
        eng = Engine.from_model_dir(folder, EngineConfig(dtype="bfloat16", page_size=16, max_cache_tokens=1024,
                                                         hip_graph=hip_graph, hip_graph_cache_size=2))
        at = [0] * 4
        outs = []

        def feed(parts):
            entries = []
            for r, n in parts:
                entries.append(StepEntry(r, seqs[r][at[r]:at[r] + n], [n - 1]))
                at[r] += n
            outs.append(eng.step(entries).cpu())
        for r in range(4):
            feed([(r, 20 + 7 * r)])
        for batch in (1, 2, 3, 1, 4, 2, 1, 3):            # four shapes over two kept graphs
            for _ in range(2):
                feed([(r, 1) for r in range(batch)])
        return outs, eng

    eager, _ = play(False)
    replayed, eng = play(True)
    assert len(eng._graphs._graphs) == 2 and eng._graphs.evictions >= 4
    assert eng._graphs.captures == 2 + eng._graphs.evictions
    for a, b in zip(eager, replayed):
        assert torch.equal(a, b)


def test_a_group_with_a_window_gets_a_pool_of_its_own_size(gpu):
    """Tiny C keeps every key in two layers and the last 24 in the other two: with at most 3 requests fed at most
    16 tokens at a time the windowed group needs 3 * (ceil((16 + 23) / 8) + 1) = 18 pages whatever the pool of the
    other group holds.  Requests longer than that run through it, against the plain implementation."""
    from prelude_amd.config import EngineConfig
    from prelude_amd.engine import Engine, StepEntry
    folder, cfg, _ = model_folder("c")
    eng = Engine.from_model_dir(folder, EngineConfig(dtype="float32", page_size=8, max_cache_tokens=1024,
                                                     max_running_requests=3, max_num_batched_tokens=16))
    windows = [g.window for g in eng.group_specs]
    assert sorted(windows) == [0, 24]
    full, windowed = windows.index(0), windows.index(24)
    assert eng.pages_per_group[full] == 128 and eng.pages_per_group[windowed] == 18
    assert eng.caches[0].k.shape[0] == 128 and eng.caches[-1].k.shape[0] == 18
    lens = [300, 210, 150]
    seqs = [reference_logits("c", 60 + i, n) for i, n in enumerate(lens)]
    got = [[] for _ in lens]
    at = [0] * 3
    rng = np.random.default_rng(2)
    while any(a < n for a, n in zip(at, lens)):
        entries, budget = [], 16
        for r in range(3):
            left = lens[r] - at[r]
            if left and budget:
                n = int(min(left, budget, rng.integers(1, 9)))
                entries.append(StepEntry(r, seqs[r][0][at[r]:at[r] + n], list(range(n))))
                budget -= n
        out = eng.step(entries).cpu()
        row = 0
        for e in entries:
            got[e.id].append(out[row:row + len(e.tokens)])
            row += len(e.tokens)
            at[e.id] += len(e.tokens)
        assert eng.tables.audit() == ""
        assert all(eng.tables.live_pages(r, windowed) <= 6 for r in range(3))
    for r in range(3):
        check(torch.cat(got[r]), seqs[r][1], "float32", f"request {r}")
    # a step beyond what the pools were sized for is refused before anything is taken
    from prelude_amd.engine import StepError
    with pytest.raises(StepError, match="max_num_batched_tokens is 16"):
        eng.step([StepEntry(9, list(range(17)), [])])
    assert not eng.has(9)
