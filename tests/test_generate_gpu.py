"""Generation through the Python entry point and the command line, against the plain implementation."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_model as pm
from helpers import PAGE, model_folder, tolerance

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def prompts_for(cfg, lengths, seed):
    g = torch.Generator().manual_seed(seed)
    return [torch.randint(0, cfg["vocab_size"] - 3, (n,), generator=g).tolist() for n in lengths]


def test_greedy_tiny_a(gpu):
    """Tiny A: prompts of 5, 17 and 31 tokens, 16 greedy steps, float32."""
    from prelude_amd import LLM
    folder, cfg, w = model_folder("a")
    prompts = prompts_for(cfg, [5, 17, 31], 0)
    llm = LLM(folder, dtype="float32", page_size=PAGE["a"], max_cache_tokens=512)
    outs = llm.generate(prompts, max_tokens=16, temperature=0.0)
    for p, o in zip(prompts, outs):
        want = pm.greedy(cfg, w, p, len(o.token_ids))
        assert o.token_ids == want
        assert o.finish_reason == ("eos" if o.token_ids[-1] == 255 else "length")
        assert o.finish_reason == "eos" or len(o.token_ids) == 16
        assert o.usage == {"prompt_tokens": len(p), "completion_tokens": len(o.token_ids), "total_tokens": len(p) + len(o.token_ids)}
        assert set(o.metrics) == {"ttft_ms", "prefill_ms", "decode_ms", "total_ms"} and o.metrics["total_ms"] > 0
    assert llm.engine.tables.audit() == "" and llm.engine.tables.num_requests() == 0


def test_temperature_tiny_b(gpu):
    """Tiny B: prompts of 1, 9, 40, 63 and 100 tokens, 24 steps at temperature 0.8, seeded: every token is the
    plain draw from the plain logits at the request's own random number."""
    from prelude_amd import LLM
    from prelude_amd.sampling import RequestSampler, SamplingParams
    folder, cfg, w = model_folder("b")
    prompts = prompts_for(cfg, [1, 9, 40, 63, 100], 1)
    llm = LLM(folder, dtype="float32", page_size=PAGE["b"], max_cache_tokens=1024, max_num_batched_tokens=64)
    outs = llm.generate(prompts, max_tokens=24, temperature=0.8, seed=7)
    again = llm.generate(prompts, max_tokens=24, temperature=0.8, seed=7)
    assert [o.token_ids for o in outs] == [o.token_ids for o in again]                # same seed, same tokens
    other = llm.generate(prompts, max_tokens=24, temperature=0.8, seed=8)
    assert [o.token_ids for o in outs] != [o.token_ids for o in other]
    checked = 0
    for p, o in zip(prompts, outs):
        rs = RequestSampler(SamplingParams(0.8, 1.0, None, 7))
        seq = list(p)
        for tok in o.token_ids:
            u = rs.next_uniform()
            prs = pm.sampling_probs(pm.forward(cfg, w, seq)[-1], 0.8)
            cdf = torch.cumsum(prs, 0)
            assert prs[tok] > 0
            if float((cdf - u * float(cdf[-1])).abs().min()) > 1e-4:
                assert tok == pm.draw(prs, u)
                checked += 1
            seq.append(tok)
        assert len(o.token_ids) == 24 or o.token_ids[-1] in (507, 508)
    assert checked > 60


def test_top_k_top_p_and_stops(gpu):
    from prelude_amd import LLM
    folder, cfg, w = model_folder("b")
    llm = LLM(folder, dtype="float32", page_size=16, max_cache_tokens=512)
    p = prompts_for(cfg, [12], 2)[0]
    greedy = llm.generate([p], max_tokens=10, temperature=0.0)[0].token_ids
    assert llm.generate([p], max_tokens=10, temperature=1.0, top_k=1, seed=3)[0].token_ids == greedy   # top-1 is greedy
    assert llm.generate([p], max_tokens=10, temperature=1.0, top_p=1e-6, seed=3)[0].token_ids == greedy
    assert llm.generate([p], max_tokens=10, temperature=1e-9, seed=3)[0].token_ids == greedy        # T -> 0
    stop = llm.generate([p], max_tokens=10, temperature=0.0, stop_token_ids=[greedy[3]])[0]
    first = greedy.index(greedy[3])
    assert stop.finish_reason == "stop" and stop.token_ids == greedy[:first + 1]                     # the stop token is kept
    assert llm.generate(p, max_tokens=3, temperature=0.0)[0].finish_reason == "length"               # a single prompt
    with pytest.raises(ValueError, match="empty"):
        llm.generate([[]])
    with pytest.raises(ValueError, match="vocabulary"):
        llm.generate([[509]])
    with pytest.raises(ValueError, match="positions"):
        llm.generate([[1] * 256])
    # max_tokens is clamped to the positions left (crates/prelude-core/src/engine/model_runner/generate.rs:23-26)
    o = llm.generate([[1] * 250], max_tokens=100, temperature=0.0, stop_token_ids=[])[0]
    assert len(o.token_ids) <= 6


def test_eos_ends_a_request(gpu, tmp_path):
    from prelude_amd import LLM
    from prelude_amd.weights import write_safetensors
    folder, cfg, w = model_folder("a")
    p = prompts_for(cfg, [9], 3)[0]
    greedy = pm.greedy(cfg, w, p, 6)
    cfg2 = dict(cfg, eos_token_id=[greedy[2], 3])
    (tmp_path / "config.json").write_text(json.dumps(cfg2))
    write_safetensors(str(tmp_path / "model.safetensors"), w)
    o = LLM(str(tmp_path), dtype="float32", page_size=8, max_cache_tokens=256).generate([p], max_tokens=6, temperature=0.0)[0]
    first = greedy.index(greedy[2])
    assert o.finish_reason == "eos" and o.token_ids == greedy[:first + 1]


def test_running_out_of_pages_changes_no_token(gpu):
    """A cache too small for all requests at once: some are evicted and recomputed, prompt and generated tokens
    alike; the tokens are those of an ample cache."""
    from prelude_amd import LLM
    folder, cfg, w = model_folder("c")
    prompts = prompts_for(cfg, [40, 70, 25, 90, 55, 33], 4)
    ample = LLM(folder, dtype="float32", page_size=8, max_cache_tokens=4096).generate(prompts, max_tokens=40, temperature=0.0)
    tight = LLM(folder, dtype="float32", page_size=8, max_cache_tokens=200, decode_reservation_cap=1,
                max_num_batched_tokens=48)
    outs = tight.generate(prompts, max_tokens=40, temperature=0.0)
    assert [o.token_ids for o in outs] == [o.token_ids for o in ample]
    assert tight.scheduler.preemptions > 0 and sum(o.preemptions for o in outs) == tight.scheduler.preemptions
    assert tight.engine.tables.audit() == "" and tight.engine.tables.num_requests() == 0
    for p, o in zip(prompts[:2], outs[:2]):
        assert o.token_ids == pm.greedy(cfg, w, p, len(o.token_ids))


def test_bfloat16_generation_runs(gpu):
    from prelude_amd import LLM
    folder, cfg, w = model_folder("b", "bfloat16")
    prompts = prompts_for(cfg, [30, 5], 5)
    outs = LLM(folder, dtype="bfloat16", page_size=16, max_cache_tokens=512).generate(prompts, max_tokens=12, temperature=0.0)
    for p, o in zip(prompts, outs):
        # every chosen token is the plain argmax, or its plain logit lies within the rounding of two bfloat16
        # logits (the chosen one's and the largest one's) of the largest
        seq = list(p)
        for tok in o.token_ids:
            lg = pm.forward(cfg, w, seq)[-1]
            assert float(lg.max() - lg[tok]) <= 2 * tolerance("bfloat16", lg), (len(seq), tok, int(lg.argmax()))
            seq.append(tok)
        assert len(o.token_ids) == 12


def test_command_line(gpu, tmp_path):
    folder, cfg, w = model_folder("a")
    p = prompts_for(cfg, [7], 6)[0]
    cmd = [sys.executable, "-m", "prelude_amd", "--model", folder, "--dtype", "f32", "--prompt-ids",
           ",".join(map(str, p)), "--max-tokens", "5", "--temperature", "0", "--page-size", "8", "--max-cache-tokens", "256"]
    r = subprocess.run(cmd, capture_output=True, text=True, cwd=ROOT, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    rec = json.loads(r.stdout.strip().splitlines()[-1])
    assert rec["token_ids"] == pm.greedy(cfg, w, p, len(rec["token_ids"])) and rec["finish_reason"] in ("length", "eos")
    assert rec["usage"]["prompt_tokens"] == 7
    # --random-weights needs only a config.json
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    cmd = [os.path.join(ROOT, "bin", "prelude-amd"), "--model", str(tmp_path), "--random-weights", "--weights-seed", "3",
           "--prompt-len", "9", "--prompt-len", "4", "--max-tokens", "4", "--temperature", "0.8", "--seed", "1",
           "--page-size", "8", "--max-cache-tokens", "256"]
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    recs = [json.loads(l) for l in r.stdout.strip().splitlines()]
    assert len(recs) == 2 and all(1 <= len(x["token_ids"]) <= 4 for x in recs)


def test_overlapped_steps_change_no_token(gpu, tmp_path):
    """Steps launched before the previous step's ids reach the host give the tokens, finish reasons and counts of
    the loop that waits for every step: with requests ending on EOS, on a stop id and on their length at
    different times, few pages (evictions), and prompts cut into portions.  In float32, where a row's logits
    are the same bits whatever else is in its step (the two loops put different requests side by side)."""
    dtype = "float32"
    from prelude_amd import LLM
    from prelude_amd.sampling import SamplingParams
    from prelude_amd.weights import write_safetensors
    folder, cfg, w = model_folder("c", dtype)
    prompts = prompts_for(cfg, [40, 70, 25, 90, 55, 33, 8], 11)
    write_safetensors(str(tmp_path / "model.safetensors"), w)
    (tmp_path / "config.json").write_text(json.dumps(dict(cfg, eos_token_id=cfg["vocab_size"] - 1)))
    probe = LLM(str(tmp_path), dtype=dtype, page_size=8, max_cache_tokens=4096, overlap_steps=False)
    base = probe.generate(prompts, max_tokens=30, temperature=0.0)
    del probe
    # an EOS id that request 0 produces midway, a stop id that request 2 produces (both greedy below)
    eos, stop = base[0].token_ids[9], base[2].token_ids[14]
    (tmp_path / "config.json").write_text(json.dumps(dict(cfg, eos_token_id=[eos])))
    params = [SamplingParams(0.0 if i % 2 == 0 else 0.9, 0.95 if i == 5 else 1.0, 20 if i == 3 else None, 100 + i)
              for i in range(len(prompts))]
    runs = []
    for overlap in (False, True):
        llm = LLM(str(tmp_path), dtype=dtype, page_size=8, max_cache_tokens=200, decode_reservation_cap=1,
                  max_num_batched_tokens=48, overlap_steps=overlap)
        outs = llm.generate(prompts, max_tokens=30, sampling_params=params, stop_token_ids=[stop])
        assert llm.engine.tables.audit() == "" and llm.engine.tables.num_requests() == 0
        assert llm.scheduler.num_running == 0 and llm.scheduler.num_waiting == 0
        runs.append((llm, outs))
    (sync_llm, sync), (over_llm, over) = runs
    assert [o.token_ids for o in over] == [o.token_ids for o in sync]
    assert [o.finish_reason for o in over] == [o.finish_reason for o in sync]
    assert sync[0].finish_reason == "eos" and sync[2].finish_reason in ("stop", "eos")
    assert "length" in {o.finish_reason for o in sync}
    assert all(len(o.token_ids) <= 30 and None not in o.token_ids for o in over)
    assert sync_llm.scheduler.preemptions > 0 and over_llm.scheduler.preemptions > 0
    assert over_llm.steps <= sync_llm.steps + 3


@pytest.mark.parametrize("seed", list(range(int(os.environ.get("PRELUDE_AMD_DRAWN_WORKLOADS", "6")))))   # widen for a hunt
def test_drawn_workloads_change_no_token(gpu, seed):
    """Requests, limits and cache sizes drawn at random: however the scheduler cuts, batches, evicts and overlaps,
    every request gets the tokens it gets when it runs in an ample cache, greedy or with its own seeded draws."""
    import numpy as np
    from prelude_amd import LLM
    from prelude_amd.sampling.sampler import SamplingParams
    rng = np.random.default_rng(seed)
    name = ["a", "b", "c"][seed % 3]
    folder, cfg, _ = model_folder(name)
    page = int(rng.choice([4, 8, 16]))
    n = int(rng.integers(3, 11))
    room = cfg["max_position_embeddings"]
    lengths = [int(rng.integers(1, min(120, room - 45))) for _ in range(n)]
    prompts = prompts_for(cfg, lengths, 50 + seed)
    max_new = int(rng.integers(1, 41))
    params = [SamplingParams(temperature=0.0) if rng.random() < 0.5 else
              SamplingParams(temperature=float(rng.choice([0.6, 1.0])), top_k=int(rng.choice([0, 5])) or None,
                             top_p=float(rng.choice([1.0, 0.9])), seed=int(rng.integers(0, 1000))) for _ in range(n)]
    ample = LLM(folder, dtype="float32", page_size=page, max_cache_tokens=8192, overlap_steps=False)
    want = ample.generate(prompts, max_tokens=max_new, sampling_params=params)
    longest = -(-(max(lengths) + max_new) // page) * page
    total = sum(-(-(m + max_new) // page) * page for m in lengths)
    tight = LLM(folder, dtype="float32", page_size=page,
                max_cache_tokens=int(rng.integers(longest + page, max(longest + 2 * page, total))),
                decode_reservation_cap=int(rng.choice([0, 1, 8])), max_num_batched_tokens=int(rng.choice([16, 48, 128])),
                long_prefill_token_threshold=int(rng.choice([0, 8, 32])), max_running_requests=int(rng.integers(2, 9)),
                overlap_steps=bool(rng.integers(0, 2)))
    got = tight.generate(prompts, max_tokens=max_new, sampling_params=params)
    for i, (g, w_) in enumerate(zip(got, want)):
        assert g.token_ids == w_.token_ids and g.finish_reason == w_.finish_reason, \
            f"seed {seed}, request {i} of {n}: {g.token_ids} ({g.finish_reason}) against {w_.token_ids} ({w_.finish_reason})"
    assert tight.engine.tables.audit() == "" and tight.engine.tables.num_requests() == 0


@pytest.mark.parametrize("seed", list(range(int(os.environ.get("PRELUDE_AMD_DRAWN_WORKLOADS", "6")))))   # widen for a hunt
def test_drawn_workloads_replayed_from_graphs_change_no_token(gpu, seed):
    """The same in bfloat16 with steps replayed from graphs (decode steps, and small steps with prompt portions once
    their shape has come twice) against the same engine with every step run directly: a replay gives the direct
    run's bits, so every request gets the same tokens, greedy or drawn, with overlapped steps and tokens carried
    on the device, few pages and evictions."""
    import numpy as np
    from prelude_amd import LLM
    from prelude_amd.sampling.sampler import SamplingParams
    rng = np.random.default_rng(5000 + seed)
    name = ["a", "b", "c"][seed % 3]
    folder, cfg, _ = model_folder(name)
    page = int(rng.choice([8, 16]))
    n = int(rng.integers(4, 13))
    room = cfg["max_position_embeddings"]
    # few different lengths, so that shapes of steps come back
    pool = [int(rng.integers(1, min(100, room - 45))) for _ in range(3)]
    lengths = [int(rng.choice(pool)) for _ in range(n)]
    prompts = prompts_for(cfg, lengths, 70 + seed)
    max_new = int(rng.integers(2, 30))
    params = [SamplingParams(temperature=0.0) if rng.random() < 0.5 else
              SamplingParams(temperature=float(rng.choice([0.6, 1.0])), top_k=int(rng.choice([0, 5])) or None,
                             top_p=float(rng.choice([1.0, 0.9])), seed=int(rng.integers(0, 1000))) for _ in range(n)]
    total = sum(-(-(m + max_new) // page) * page for m in lengths)
    longest = -(-(max(lengths) + max_new) // page) * page
    common = dict(dtype="bfloat16", page_size=page, max_cache_tokens=int(rng.integers(longest + page, max(longest + 2 * page, total))),
                  max_num_batched_tokens=int(rng.choice([48, 128, 512])), max_running_requests=int(rng.integers(2, 9)),
                  overlap_steps=bool(rng.integers(0, 2)))
    direct = LLM(folder, hip_graph=False, **common)
    want = direct.generate(prompts, max_tokens=max_new, sampling_params=params)
    replayed = LLM(folder, hip_graph=True, **common)
    got = replayed.generate(prompts, max_tokens=max_new, sampling_params=params)
    for i, (g, w_) in enumerate(zip(got, want)):
        assert g.token_ids == w_.token_ids and g.finish_reason == w_.finish_reason, \
            f"seed {seed}, request {i} of {n}: {g.token_ids} ({g.finish_reason}) against {w_.token_ids} ({w_.finish_reason})"
    assert replayed.engine._graphs.replays > 0
    assert replayed.engine.tables.audit() == "" and replayed.engine.tables.num_requests() == 0


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_a_session_of_arrivals_and_cancellations_replayed_from_graphs(gpu, seed):
    """One engine, some hundred requests that arrive, end and are cancelled at drawn steps, with few pages and few
    graphs kept (so graphs are dropped and captured again): with steps replayed from graphs every request ends as
    it does with every step run directly, in as many steps.  (Widened by hand to 96,000 requests in 220,000 steps
    over the three configurations: no request differs.)"""
    import numpy as np
    from prelude_amd import LLM
    from prelude_amd.sampling.sampler import SamplingParams
    folder, cfg, _ = model_folder(["a", "b", "c"][seed])
    room = cfg["max_position_embeddings"]
    count = 300

    def play(hip_graph, overlap):
        rng = np.random.default_rng(8000 + seed)
        llm = LLM(folder, dtype="bfloat16", page_size=16, max_cache_tokens=int(rng.choice([384, 640])),
                  max_num_batched_tokens=int(rng.choice([48, 128])), max_running_requests=int(rng.integers(3, 9)),
                  overlap_steps=overlap, hip_graph=hip_graph, hip_graph_cache_size=6)
        pool = [int(rng.integers(1, min(90, room - 40))) for _ in range(4)]
        session = llm.session()
        ended, added, steps = {}, 0, 0
        while added < count or session.pending:
            for _ in range(int(rng.integers(0, 3)) if added < count else 0):
                sampling = SamplingParams(temperature=0.0) if rng.random() < 0.6 else \
                    SamplingParams(temperature=0.8, top_k=5, seed=int(rng.integers(0, 999)))
                session.add(rng.integers(1, cfg["vocab_size"], size=int(rng.choice(pool))).tolist(),
                            max_tokens=int(rng.integers(1, 25)), sampling=sampling)
                added += 1
            if added and rng.random() < 0.05:
                index = int(rng.integers(0, added))
                result = session.cancel(index)
                if result is not None:
                    ended[index] = ("cancelled", tuple(result.token_ids))
            for index, result in session.step():
                ended[index] = (result.finish_reason, tuple(result.token_ids))
            steps += 1
        assert llm.engine.tables.audit() == "" and llm.engine.tables.num_requests() == 0
        return ended, steps, llm.engine._graphs

    for overlap in (False, True):
        want, direct_steps, _ = play(False, overlap)
        got, steps, graphs = play(True, overlap)
        assert steps == direct_steps and len(got) == len(want) >= count
        assert [i for i in want if want[i] != got.get(i)] == []
        assert graphs.replays > steps // 2 and graphs.evictions > 0
        assert any(reason == "cancelled" for reason, _ in want.values())


def test_tokens_are_handed_over_as_they_come(gpu):
    from prelude_amd import LLM
    folder, cfg, _ = model_folder("a")
    prompts = prompts_for(cfg, [12, 40, 3], 9)
    for overlap in (True, False):
        seen = {i: [] for i in range(3)}
        llm = LLM(folder, dtype="float32", page_size=8, max_cache_tokens=512, overlap_steps=overlap)
        outs = llm.generate(prompts, max_tokens=9, temperature=0.8, seed=5, on_token=lambda i, t: seen[i].append(t))
        assert [seen[i] for i in range(3)] == [o.token_ids for o in outs]


def test_requests_join_a_running_session(gpu):
    """Requests added while others are decoding get the tokens they get alone, and a session that is given up
    leaves nothing behind in the scheduler or the cache."""
    from prelude_amd import LLM
    from prelude_amd.sampling.sampler import SamplingParams
    folder, cfg, w = model_folder("c")
    prompts = prompts_for(cfg, [30, 8, 55, 17, 3], 12)
    llm = LLM(folder, dtype="float32", page_size=8, max_cache_tokens=1024, max_num_batched_tokens=32)
    alone = [llm.generate([p], max_tokens=20, temperature=0.0)[0].token_ids for p in prompts]
    s = llm.session()
    got, ends, steps = {}, [], 0
    arrivals = {0: [0], 3: [1, 2], 11: [3], 25: [4]}        # step -> prompts that arrive before it
    while s.pending or steps <= max(arrivals):
        for i in arrivals.get(steps, []):
            assert s.add(prompts[i], max_tokens=20, sampling=SamplingParams(temperature=0.0)) == i
        for index, res in s.step():
            got[index] = res.token_ids
            ends.append(index)
        steps += 1
    assert [got[i] for i in range(5)] == alone
    assert ends.index(1) < ends.index(4)                      # the late arrival ends after an early one
    assert llm.engine.tables.audit() == "" and llm.engine.tables.num_requests() == 0
    s = llm.session()
    s.add(prompts[2], max_tokens=50, sampling=SamplingParams(temperature=0.0))
    for _ in range(4):
        s.step()
    s.abandon()
    assert not s.pending and llm.engine.tables.num_requests() == 0 and llm.engine.tables.audit() == ""
    assert llm.generate([prompts[1]], max_tokens=20, temperature=0.0)[0].token_ids == alone[1]
    with pytest.raises(ValueError, match="prompt 1: the prompt is empty"):
        llm.generate([[1, 2], []], max_tokens=4)
    assert llm.engine.tables.num_requests() == 0


def test_text_prompts_and_stop_strings(gpu, tmp_path):
    """A folder with a tokenizer.json takes text prompts, returns text, and ends a request once its text holds a
    stop string (the text returned ends before it; the ids keep the tokens that spelt it)."""
    import shutil
    from tokenizers import Tokenizer, models, pre_tokenizers
    from prelude_amd import LLM
    folder, cfg, w = model_folder("a")
    for name in ("config.json", "model.safetensors"):
        shutil.copy(os.path.join(folder, name), tmp_path / name)
    vocab = {f"w{i}": i for i in range(cfg["vocab_size"])}
    tok = Tokenizer(models.WordLevel(vocab, unk_token="w0"))
    tok.pre_tokenizer = pre_tokenizers.Whitespace()
    tok.save(str(tmp_path / "tokenizer.json"))
    llm = LLM(str(tmp_path), dtype="float32", page_size=8, max_cache_tokens=512)
    prompt = "w5 w17 w3 w200 w41"
    free = llm.generate(prompt, max_tokens=12, temperature=0.0)[0]
    assert free.prompt_token_ids == [5, 17, 3, 200, 41]
    assert free.token_ids == pm.greedy(cfg, w, free.prompt_token_ids, len(free.token_ids))
    assert free.text == " ".join(f"w{t}" for t in free.token_ids)
    words = free.text.split()
    assert len(words) >= 6
    # the fifth word as a stop string: the request ends with the token that completes it
    at = next(i for i, x in enumerate(words) if x == words[4])
    for overlap in (True, False):
        llm2 = LLM(str(tmp_path), dtype="float32", page_size=8, max_cache_tokens=512, overlap_steps=overlap)
        cut = llm2.generate([prompt, [5, 17, 3]], max_tokens=12, temperature=0.0, stop=[words[4], "never there"])
        assert cut[0].finish_reason == "stop" and cut[0].token_ids == free.token_ids[:at + 1]
        assert cut[0].text == " ".join(words[:at]) + (" " if at else "")
        assert cut[1].finish_reason in ("length", "eos", "stop")
        assert llm2.engine.tables.audit() == "" and llm2.engine.tables.num_requests() == 0
    with pytest.raises(ValueError, match="tokenizer.json"):
        LLM(folder, dtype="float32", page_size=8, max_cache_tokens=512).generate([[1, 2]], stop=["x"])


@pytest.mark.parametrize("overlap", [True, False])
def test_logprobs_of_generated_and_prompt_tokens(gpu, overlap):
    """log P of every generated token with the k likeliest, and of every prompt token given those before it,
    against log_softmax of the plain implementation's logits; prompts cut into portions, a cache tight enough to
    evict, sampled and greedy requests side by side."""
    from prelude_amd import LLM
    from prelude_amd.sampling.sampler import SamplingParams
    folder, cfg, w = model_folder("b")
    prompts = prompts_for(cfg, [37, 9, 60, 2], 8)
    params = [SamplingParams(temperature=0.0), SamplingParams(temperature=0.9, seed=3),
              SamplingParams(temperature=0.0), SamplingParams(temperature=0.7, top_k=5, seed=4)]
    llm = LLM(folder, dtype="float32", page_size=16, max_cache_tokens=128, max_num_batched_tokens=24,
              decode_reservation_cap=1, overlap_steps=overlap)
    outs = llm.generate(prompts, max_tokens=30, sampling_params=params, logprobs=3, prompt_logprobs=True)
    assert llm.scheduler.preemptions > 0
    for p, o in zip(prompts, outs):
        ref = torch.log_softmax(pm.forward(cfg, w, p + o.token_ids), dim=-1)
        n = len(p)
        assert len(o.token_logprobs) == len(o.token_ids) == len(o.top_logprobs)
        for i, tok in enumerate(o.token_ids):
            row = ref[n - 1 + i]
            assert abs(o.token_logprobs[i] - float(row[tok])) < 1e-4
            want = torch.topk(row, 3)
            assert [t for t, _ in o.top_logprobs[i]] == want.indices.tolist()
            assert all(abs(v - float(x)) < 1e-4 for (_, v), x in zip(o.top_logprobs[i], want.values))
        assert o.prompt_logprobs[0] is None and len(o.prompt_logprobs) == n
        for j in range(1, n):
            assert abs(o.prompt_logprobs[j] - float(ref[j - 1, p[j]])) < 1e-4, (j, n)
    plain = llm.generate(prompts[:2], max_tokens=5, temperature=0.0)
    assert plain[0].token_logprobs is None and plain[0].top_logprobs is None and plain[0].prompt_logprobs is None
    only = llm.generate(prompts[:1], max_tokens=5, temperature=0.0, logprobs=0)[0]
    assert len(only.token_logprobs) == 5 and only.top_logprobs is None
    assert llm.engine.tables.audit() == "" and llm.engine.tables.num_requests() == 0


@pytest.mark.parametrize("overlap", [True, False])
def test_one_request_is_cancelled(gpu, overlap):
    """``Session.cancel``: the request ends at once with the tokens it has and the reason ``cancelled``, what it
    held goes back, and the others generate what they generate alone."""
    from prelude_amd import LLM, SamplingParams
    folder, cfg, w = model_folder("a")
    prompts = prompts_for(cfg, [20, 33, 9], 7)
    llm = LLM(folder, dtype="float32", page_size=8, max_cache_tokens=1024, overlap_steps=overlap)
    alone = llm.generate(prompts, max_tokens=30, temperature=0.0)
    s = llm.session()
    idx = [s.add(p, max_tokens=30, sampling=SamplingParams(temperature=0.0)) for p in prompts]
    results, steps = {}, 0
    while s.pending:
        for i, res in s.step():
            results[i] = res
        steps += 1
        if steps == 6:
            res = s.cancel(idx[1])
            assert res.finish_reason == "cancelled" and res.error is None
            assert 0 < len(res.token_ids) < 30 and res.token_ids == alone[1].token_ids[:len(res.token_ids)]
            assert s.cancel(idx[1]) is None                      # it is gone
            assert llm.engine.tables.audit() == "" and llm.engine.tables.num_requests() == 2
    assert sorted(results) == [idx[0], idx[2]]
    for i in (0, 2):
        assert results[idx[i]].token_ids == alone[i].token_ids and results[idx[i]].finish_reason == alone[i].finish_reason
    assert llm.engine.tables.audit() == "" and llm.engine.tables.num_requests() == 0
    # a request that has not run yet can be cancelled too
    s = llm.session()
    a = s.add(prompts[0], max_tokens=5, sampling=SamplingParams(temperature=0.0))
    b = s.add(prompts[2], max_tokens=5, sampling=SamplingParams(temperature=0.0))
    res = s.cancel(b)
    assert res.finish_reason == "cancelled" and res.token_ids == []
    out = {}
    while s.pending:
        out.update(dict(s.step()))
    assert list(out) == [a] and out[a].token_ids == alone[0].token_ids[:5]


@pytest.mark.parametrize("overlap", [True, False])
def test_a_failed_step_ends_its_requests_and_no_others(gpu, overlap):
    """A step that cannot be run (here: the engine's run is made to raise once) ends every request of that step
    with the reason ``error`` and what they held goes back (crates/prelude-core/src/engine/run/ar.rs:1647-1665);
    requests that were not in it go on and generate what they generate alone."""
    from prelude_amd import LLM
    folder, cfg, w = model_folder("a")
    prompts = prompts_for(cfg, [20, 33, 9, 14], 8)
    llm = LLM(folder, dtype="float32", page_size=8, max_cache_tokens=1024, overlap_steps=overlap, max_running_requests=2)
    alone = llm.generate(prompts, max_tokens=12, temperature=0.0)
    real_run = llm.engine.run
    calls = {"n": 0, "fail_at": 1}

    def run(entries, starts, carried=None):
        calls["n"] += 1
        if calls["n"] == calls["fail_at"]:
            raise RuntimeError("injected failure")
        return real_run(entries, starts, carried)

    llm.engine.run = run
    # the very first step fails: its two requests end with nothing, the two that waited run as if alone
    outs = llm.generate(prompts, max_tokens=12, temperature=0.0)
    assert [o.finish_reason for o in outs[:2]] == ["error", "error"] and all(o.token_ids == [] for o in outs[:2])
    assert all("RuntimeError: injected failure" in o.error for o in outs[:2])
    assert [o.token_ids for o in outs[2:]] == [o.token_ids for o in alone[2:]] and all(o.error is None for o in outs[2:])
    assert llm.engine.tables.audit() == "" and llm.engine.tables.num_requests() == 0
    assert llm.scheduler.num_running == 0 and llm.scheduler.num_waiting == 0
    # a decode step fails: its requests keep the tokens they had, every one of them the token of the run alone
    calls.update(n=0, fail_at=6)
    outs = llm.generate(prompts, max_tokens=12, temperature=0.0)
    assert [o.finish_reason for o in outs[:2]] == ["error", "error"]
    for o, a in zip(outs[:2], alone[:2]):
        assert 0 < len(o.token_ids) < 12 and o.token_ids == a.token_ids[:len(o.token_ids)]
    assert [o.token_ids for o in outs[2:]] == [o.token_ids for o in alone[2:]]
    assert llm.engine.tables.audit() == "" and llm.engine.tables.num_requests() == 0


def test_prompt_logprobs_are_taken_in_portions(gpu, monkeypatch):
    """With ``prompt_logprobs`` the logits of every prompt position are wanted: the request is then fed in
    portions of at most ``PROMPT_LOGPROBS_CHUNK`` tokens, so that no step holds more than that many rows of logits
    for it (crates/prelude-core/src/engine/model_runner/paged_mixed.rs:172-270); the numbers do not change."""
    import prelude_amd.llm as L
    from prelude_amd import LLM
    folder, cfg, w = model_folder("b")
    prompts = prompts_for(cfg, [70, 11], 9)
    llm = LLM(folder, dtype="float32", page_size=16, max_cache_tokens=1024)
    whole = llm.generate(prompts, max_tokens=3, temperature=0.0, prompt_logprobs=True)
    monkeypatch.setattr(L, "PROMPT_LOGPROBS_CHUNK", 16)
    seen = []
    real_run = llm.engine.run
    llm.engine.run = lambda entries, starts, carried=None: (seen.append([len(e.want) for e in entries]),
                                                            real_run(entries, starts, carried))[1]
    cut = llm.generate(prompts, max_tokens=3, temperature=0.0, prompt_logprobs=True)
    assert max(max(s) for s in seen) <= 16 and len(seen) >= 5
    for a, b in zip(whole, cut):
        assert a.token_ids == b.token_ids
        assert a.prompt_logprobs[0] is None and b.prompt_logprobs[0] is None
        assert np.allclose(a.prompt_logprobs[1:], b.prompt_logprobs[1:], atol=2e-5)
