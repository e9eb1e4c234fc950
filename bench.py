#!/usr/bin/env python3
"""Decode and prefill throughput of the engine on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--context 4096]

The default run has the layer sizes of the Qwen3-4B shape (36 layers, hidden
2560, 32 heads, 8 KV heads, head_dim 128, intermediate 9728, vocabulary
151936, tied head) with random bfloat16 weights, a batch of 8 and a context of
4,096 tokens: every request is prefilled through the engine's own step
function, then K decode steps are timed (each step: build the batch, run the
model from the paged cache, greedy argmax on the device, ids back to the host;
the host prepares a step while the one before it runs, as the engine's
generation loop does).
One JSON line is printed: ``value`` is decoded tokens a second; ``prefill`` is
a 2,048-token prompt portion (the median of its repetitions); ``roofline`` prices
the decode step against HBM bandwidth; ``points`` holds, in tokens a second each:
batch 1, 32 and 64 at the same context; batch 64 again on a pool whose pages were
handed out, given back and handed out again in a random order of requests
(``decode_b64_churned``); batch 8 at a context of 32,768 tokens; prompts of 256,
512 and 8,192 tokens in one step; and at the other shapes the benchmark
configurations name: batch 8 and a 2,048-token prompt at the 8B shape, a step of
a 2,048-token portion beside 63 decoding requests at contexts up to 8,192 there
(``8b_mixed_2048+63``), and batch 8 at the 32B shape.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0           # MI355X HBM3E
MFMA_PEAK = {"bf16": 2.5e15, "fp16": 2.5e15, "fp8": 5.0e15, "f32": 157.3e12}

QWEN3_4B = dict(architectures=["Qwen3ForCausalLM"], model_type="qwen3", vocab_size=151936, hidden_size=2560,
                intermediate_size=9728, num_hidden_layers=36, num_attention_heads=32, num_key_value_heads=8,
                head_dim=128, attention_bias=False, max_position_embeddings=40960, sliding_window=None,
                max_window_layers=36, tie_word_embeddings=True, rope_theta=1000000.0, rms_norm_eps=1e-6,
                use_sliding_window=False, hidden_act="silu", eos_token_id=151645)


# the other shapes the benchmark configurations name (not the default run): --shape 8b | 32b
QWEN3_8B = dict(QWEN3_4B, hidden_size=4096, intermediate_size=12288, tie_word_embeddings=False)
QWEN3_32B = dict(QWEN3_4B, hidden_size=5120, intermediate_size=25600, num_hidden_layers=64, num_attention_heads=64,
                 max_window_layers=64, tie_word_embeddings=False)
QWEN3_06B = dict(QWEN3_4B, hidden_size=1024, intermediate_size=3072, num_hidden_layers=28, num_attention_heads=16,
                 max_window_layers=28)
SHAPES = {"0.6b": QWEN3_06B, "4b": QWEN3_4B, "8b": QWEN3_8B, "32b": QWEN3_32B}


def build_engine(raw, dtype, cache_tokens, seed=0, page_size=16, **cfg_overrides):
    """The engine in its random-weights mode: the product's own loader, tensors drawn on the device."""
    from prelude_amd.config import EngineConfig
    from prelude_amd.engine import Engine
    cfg = EngineConfig(dtype=dtype, page_size=page_size, max_cache_tokens=cache_tokens, **cfg_overrides)
    return Engine.from_config(raw, cfg, seed=seed)


def release_memory():
    """Gives the last engine's device memory back before the next engine is built (the caller has dropped it)."""
    import gc
    import torch
    gc.collect()
    torch.cuda.empty_cache()


def weight_bytes(raw, el):
    h, i, v = raw["hidden_size"], raw["intermediate_size"], raw["vocab_size"]
    nh, nkv, hd, L = raw["num_attention_heads"], raw["num_key_value_heads"], raw["head_dim"], raw["num_hidden_layers"]
    per_layer = ((nh + 2 * nkv) * hd * h + nh * hd * h + 3 * i * h) * el + (2 * h + 2 * hd) * 4
    head = v * h * el           # the head matrix is read whole; the embedding (the same matrix when tied) only gathers rows
    return L * per_layer + head + h * 4, L * ((nh + 2 * nkv) * hd * h + nh * hd * h + 3 * i * h)


def kv_bytes_per_token(raw, el):
    return raw["num_hidden_layers"] * 2 * raw["num_key_value_heads"] * raw["head_dim"] * el


def prefill_requests(engine, batch, length, chunk, vocab, seed):
    import numpy as np
    from prelude_amd.engine import StepEntry
    rng = np.random.default_rng(seed)
    prompts = [rng.integers(0, vocab, size=length).tolist() for _ in range(batch)]
    for rid, p in enumerate(prompts):
        for s in range(0, length, chunk):
            engine.step([StepEntry(rid, p[s:s + chunk], [])])
    return prompts


def time_decode(engine, batch, steps, warmup, vocab, ids=None):
    """Greedy decode steps for `batch` live requests; returns seconds per step.

    As in ``LLM.generate``, a step is launched with the previous step's ids
    still on the device, and those ids are read on the host while it runs.
    """
    import torch
    from prelude_amd.engine import StepEntry
    from prelude_amd.ops import kernels as K
    state = {"sampled": None, "pending": None, "ids": [1] * batch}
    rids = list(range(batch)) if ids is None else list(ids)

    def one():
        prev = state["sampled"]
        if prev is None:
            entries = [StepEntry(rids[r], [state["ids"][r]], [0]) for r in range(batch)]
        else:
            entries = [StepEntry(rids[r], [0], [0], carry=r) for r in range(batch)]
        logits = engine.step(entries, carried=prev)
        sampled = K.argmax(logits)
        host = torch.empty(batch, dtype=torch.int32, pin_memory=True)
        host.copy_(sampled, non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        if state["pending"] is not None:
            pev, phost = state["pending"]
            pev.synchronize()
            state["ids"] = phost.tolist()
        state["sampled"], state["pending"] = sampled, (ev, host)

    for _ in range(warmup):
        one()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        one()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def churned_requests(engine, batch, length, vocab, seed):
    """`batch` live requests of `length` tokens on a pool that has been through a session: requests of random
    lengths are admitted in turn, a random half of them ends, others take their pages, and every request grows in
    portions of random size in a random order of requests, so that no request's pages lie in one run."""
    import numpy as np
    from prelude_amd.engine import StepEntry
    rng = np.random.default_rng(seed)
    have = {}
    next_id = 0

    def grow(rid, upto):
        while have[rid] < upto:
            n = int(min(upto - have[rid], rng.integers(48, 400)))
            engine.step([StepEntry(rid, rng.integers(0, vocab, size=n).tolist(), [])])
            have[rid] += n
            yield

    for _ in range(3):                                   # three generations of requests
        while len(have) < batch:
            have[next_id] = 0
            next_id += 1
        growers = [grow(rid, int(rng.integers(length // 4, length))) for rid in have]
        while growers:                                   # all of them grow, a portion at a time, in random order
            i = int(rng.integers(0, len(growers)))
            if next(growers[i], "done") == "done":
                growers.pop(i)
        for rid in rng.permutation(list(have))[: batch // 2].tolist():
            engine.release(rid)
            del have[rid]
    while len(have) < batch:
        have[next_id] = 0
        next_id += 1
    growers = [grow(rid, length) for rid in have]
    while growers:
        i = int(rng.integers(0, len(growers)))
        if next(growers[i], "done") == "done":
            growers.pop(i)
    return sorted(have)


def decode_point(raw, dtype, batch, context, steps, warmup, layers_note, chunk=2048, churned=False):
    import torch
    total = steps + warmup
    eng = build_engine(raw, dtype, cache_tokens=batch * (context + 64), max_num_batched_tokens=max(8192, chunk))
    if churned:
        ids = churned_requests(eng, batch, context - total, raw["vocab_size"], seed=batch)
        sec = time_decode(eng, batch, steps, warmup, raw["vocab_size"], ids)
        del eng
        release_memory()
        return sec
    prefill_requests(eng, batch, context - total, chunk, raw["vocab_size"], seed=batch)
    sec = time_decode(eng, batch, steps, warmup, raw["vocab_size"])
    del eng
    release_memory()
    return sec


def time_prefill(raw, dtype, tokens, reps):
    """Seconds a prompt of `tokens` tokens takes in one step, its last logits wanted: the median of `reps` runs."""
    import numpy as np
    import torch
    from prelude_amd.engine import StepEntry
    eng = build_engine(raw, dtype, cache_tokens=(reps + 2) * (tokens + 64), max_num_batched_tokens=max(8192, tokens))
    rng = np.random.default_rng(7)
    times = []
    for r in range(reps + 1):
        p = rng.integers(0, raw["vocab_size"], size=tokens).tolist()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        eng.step([StepEntry(100 + r, p, [tokens - 1])])
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        eng.release(100 + r)
        if r > 0:
            times.append(dt)
    del eng
    release_memory()
    return sorted(times)[len(times) // 2]           # the median (the first run, which sets things up, left out)


def time_mixed(raw, dtype, chunk, decoding, context, steps, warmup):
    """A step with one prompt portion of `chunk` tokens beside `decoding` requests that feed one token each, at
    contexts spread up to `context`; the portion continues a prompt that is already `context - chunk` long.
    Returns seconds per step."""
    import numpy as np
    import torch
    from prelude_amd.engine import StepEntry
    total = steps + warmup
    rng = np.random.default_rng(11)
    vocab = raw["vocab_size"]
    lens = [int(x) for x in np.linspace(256, context - total - 1, decoding)]
    need = sum(-(-(n + total + 1) // 64) * 64 for n in lens) + total * (context + 64)
    eng = build_engine(raw, dtype, cache_tokens=need + 4096)
    for rid, n in enumerate(lens):
        p = rng.integers(0, vocab, size=n).tolist()
        for s0 in range(0, n, 2048):
            eng.step([StepEntry(rid, p[s0:s0 + 2048], [])])
    times = []
    for it in range(total):
        big = 1000 + it
        head = rng.integers(0, vocab, size=context - chunk).tolist()
        for s0 in range(0, len(head), 2048):
            eng.step([StepEntry(big, head[s0:s0 + 2048], [])])
        entries = [StepEntry(big, rng.integers(0, vocab, size=chunk).tolist(), [chunk - 1])]
        entries += [StepEntry(rid, [int(rng.integers(0, vocab))], [0]) for rid in range(decoding)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        eng.step(entries)
        torch.cuda.synchronize()
        times.append(time.perf_counter() - t0)
        eng.release(big)
    del eng
    release_memory()
    return sum(times[warmup:]) / steps


def time_requests(raw, dtype, requests, prompt_len, max_tokens, concurrency, **cfg_overrides):
    """`requests` prompts of `prompt_len` random tokens, `max_tokens` new tokens each, through an LLM session
    that is kept at `concurrency` requests: whenever one ends the next is added, as a load generator with that
    many clients does (the reference's published workload is this with one new token, over HTTP).
    Returns (seconds in all, sorted list of seconds from a request's arrival to its end)."""
    import numpy as np
    from prelude_amd import LLM, SamplingParams
    eng = build_engine(raw, dtype, cache_tokens=min(requests, max(concurrency, 16)) * (prompt_len + max_tokens + 64),
                       **cfg_overrides)
    llm = LLM.from_engine(eng)
    rng = np.random.default_rng(5)
    prompts = [rng.integers(0, raw["vocab_size"] - 1000, size=prompt_len).tolist() for _ in range(requests)]
    llm.generate(prompts[:min(concurrency, 8)], max_tokens=max_tokens, temperature=0.0)   # warm-up
    greedy = SamplingParams(temperature=0.0)
    session = llm.session()
    sent, latencies, firsts = 0, [], []
    t0 = time.perf_counter()
    while sent < min(concurrency, requests):
        session.add(prompts[sent], max_tokens=max_tokens, sampling=greedy)
        sent += 1
    while session.pending:
        for _, res in session.step():
            latencies.append(res.metrics["total_ms"] / 1e3)
            firsts.append(res.metrics["ttft_ms"] / 1e3)
            if sent < requests:
                session.add(prompts[sent], max_tokens=max_tokens, sampling=greedy)
                sent += 1
    return time.perf_counter() - t0, sorted(latencies), sorted(firsts)


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the configuration has (named in config)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--shape", default="4b", choices=sorted(SHAPES), help="layer sizes: Qwen3-4B (the default run), 0.6B, 8B or 32B")
    ap.add_argument("--prefill-tokens", type=int, default=2048)
    ap.add_argument("--no-points", action="store_true", help="skip the points at other batches and lengths")
    ap.add_argument("--no-prefill", action="store_true")
    ap.add_argument("--prefill-only", action="store_true", help="time the prefill alone and print its record (for profiles)")
    ap.add_argument("--mixed", action="store_true",
                    help="time a step of one --prefill-tokens portion beside 63 decoding requests at contexts up to "
                         "--context, and print its record")
    ap.add_argument("--requests", type=int, default=0,
                    help="time this many prompts (--prompt-len tokens, --new-tokens new tokens each) through "
                         "LLM.generate, --concurrency at a time, and print the record")
    ap.add_argument("--concurrency", type=int, default=96)
    ap.add_argument("--graph-portion-tokens", type=int, default=None,
                    help="--requests: steps with prompt portions of up to this many tokens are replayed from graphs "
                         "(0: never; default: the engine's own)")
    ap.add_argument("--prompt-len", type=int, default=512, help="prompt length of --requests")
    ap.add_argument("--new-tokens", type=int, default=1, help="new tokens per request of --requests")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this engine runs on one GPU; --gpus %d is not supported" % args.gpus, flush=True)
        return 2

    import torch
    raw = dict(SHAPES[args.shape])
    name = f"Qwen3-{args.shape.upper()} shape"
    full_layers = raw["num_hidden_layers"]
    if args.layers:
        raw["num_hidden_layers"] = args.layers
        raw["max_window_layers"] = args.layers
    el = 2 if args.dtype == "bfloat16" else 4
    short = "bf16" if args.dtype == "bfloat16" else "f32"

    if args.mixed:
        sec = time_mixed(raw, args.dtype, args.prefill_tokens, 63, args.context, max(4, args.steps // 8), 2)
        toks = args.prefill_tokens + 63
        print(json.dumps({"model": name, "mixed_step": f"{args.prefill_tokens} prompt tokens + 63 decoding requests",
                          "context": args.context, "ms": round(sec * 1e3, 3), "tok_per_s": round(toks / sec, 1)}),
              flush=True)
        return 0
    if args.requests:
        over = {} if args.graph_portion_tokens is None else {"hip_graph_portion_tokens": args.graph_portion_tokens}
        total, calls, firsts = time_requests(raw, args.dtype, args.requests, args.prompt_len, args.new_tokens,
                                             args.concurrency, **over)
        mean = lambda v: sum(v) / len(v)
        tpot = (mean(calls) - mean(firsts)) / max(args.new_tokens - 1, 1)
        print(json.dumps({"model": name, "workload": f"{args.requests} prompts of {args.prompt_len} tokens, "
                          f"{args.new_tokens} new token(s), {args.concurrency} at a time (LLM session, no HTTP)",
                          "req_per_s": round(args.requests / total, 1),
                          "prompt_tok_per_s": round(args.requests * args.prompt_len / total, 1),
                          "new_tok_per_s": round(args.requests * args.new_tokens / total, 1),
                          "ttft_ms_mean": round(mean(firsts) * 1e3, 2), "tpot_ms_mean": round(tpot * 1e3, 3),
                          "latency_ms_mean": round(mean(calls) * 1e3, 2),
                          "latency_ms_p50": round(calls[len(calls) // 2] * 1e3, 2),
                          "latency_ms_p95": round(calls[min(len(calls) - 1, int(len(calls) * 0.95))] * 1e3, 2)}),
              flush=True)
        return 0
    if args.prefill_only:
        psec = time_prefill(raw, args.dtype, args.prefill_tokens, reps=5)
        print(json.dumps({"prefill_tokens": args.prefill_tokens, "ms": round(psec * 1e3, 3),
                          "tok_per_s": round(args.prefill_tokens / psec, 1)}), flush=True)
        return 0
    sec = decode_point(raw, args.dtype, args.batch, args.context, args.steps, args.warmup, None)
    value = args.batch / sec
    wbytes, matmul_params = weight_bytes(raw, el)
    step_bytes = wbytes + args.batch * args.context * kv_bytes_per_token(raw, el)
    achieved = step_bytes / sec / 1e9

    out = {
        "metric": f"decode tok/s @ batch {args.batch}, context {args.context} ({name}, {short})",
        "value": round(value, 2), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(sec * 1e3, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": short, "data": "synthetic (random tokens, random-init weights)",
        "config": {"model": name, "layers": raw["num_hidden_layers"], "layers_full": full_layers,
                   "hidden": raw["hidden_size"], "heads": raw["num_attention_heads"],
                   "kv_heads": raw["num_key_value_heads"], "head_dim": raw["head_dim"],
                   "intermediate": raw["intermediate_size"], "vocab": raw["vocab_size"], "tied": bool(raw["tie_word_embeddings"]),
                   "global_batch": args.batch, "seq_len": args.context, "page_size": 16, "parallelism": "none"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4)},
    }
    if not args.no_prefill:
        T = args.prefill_tokens
        psec = time_prefill(raw, args.dtype, T, reps=5)
        nh, hd, L = raw["num_attention_heads"], raw["head_dim"], raw["num_hidden_layers"]
        flops = 2.0 * T * matmul_params + L * 2.0 * nh * hd * T * T + 2.0 * raw["vocab_size"] * raw["hidden_size"]
        out["prefill"] = {"value": round(T / psec, 1), "tokens": T, "ms": round(psec * 1e3, 3),
                          "frac": round(flops / psec / MFMA_PEAK[short], 4)}
    if not args.no_points:
        pts = {}
        for b in (1, 32, 64):   # 32: the products of 17 to 128 rows, where attention does not yet dominate the step
            s = decode_point(raw, args.dtype, b, args.context, max(8, args.steps // 2), max(2, args.warmup // 2), None)
            pts[f"decode_b{b}"] = round(b / s, 2)
        if args.context == 4096 and args.batch == 8:
            # further from the default point: a long context (the cache is 3.6 times the weights there) and a long portion
            s = decode_point(raw, args.dtype, 8, 32768, max(8, args.steps // 4), max(2, args.warmup // 4), None, chunk=8192)
            pts["decode_b8_ctx32768"] = round(8 / s, 2)
            s = decode_point(raw, args.dtype, 64, args.context, max(8, args.steps // 2), max(2, args.warmup // 2), None,
                             churned=True)
            pts["decode_b64_churned"] = round(64 / s, 2)
            if not args.no_prefill:
                pts["prefill_8192"] = round(8192 / time_prefill(raw, args.dtype, 8192, reps=3), 1)
                for t in (256, 512):
                    pts[f"prefill_{t}"] = round(t / time_prefill(raw, args.dtype, t, reps=5), 1)
            if args.shape == "4b" and not args.layers:
                # the other shapes the benchmark configurations name, at their own points
                big = dict(SHAPES["8b"])
                s = decode_point(big, args.dtype, 8, args.context, max(8, args.steps // 2), max(2, args.warmup // 2), None)
                pts["8b_decode_b8"] = round(8 / s, 2)
                if not args.no_prefill:
                    pts["8b_prefill_2048"] = round(2048 / time_prefill(big, args.dtype, 2048, reps=3), 1)
                s = time_mixed(big, args.dtype, 2048, 63, 8192, 4, 2)
                pts["8b_mixed_2048+63"] = round((2048 + 63) / s, 1)
                big = dict(SHAPES["32b"])
                s = decode_point(big, args.dtype, 8, args.context, max(8, args.steps // 2), max(2, args.warmup // 2), None)
                pts["32b_decode_b8"] = round(8 / s, 2)
        out["points"] = pts
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
