"""Command line: load a model folder (or make one with random weights) and generate.

Option names and meanings are the reference server's where it has them
(crates/prelude-server/src/main.rs:15-183: --model, --model-path, --dtype,
--device, --max-running-requests, --max-num-batched-tokens,
--long-prefill-token-threshold, --max-total-tokens, --decode-reservation-cap,
--decode-priority-max-remaining-tokens, --gpu-memory-utilization,
--cuda-graph/--no-cuda-graph).  The request fields the reference takes per
HTTP request are options here: --max-tokens, --temperature, --top-p, --top-k,
--seed, --stop-token-ids (crates/prelude-core/src/types.rs:63-96, :388-413).
--random-weights is ours: it needs only a config.json, and draws the tensors
on the device; with --write-model DIR the drawn model is written out as a
folder (config.json, model.safetensors) and loaded from there.
"""
from __future__ import annotations

import argparse
import json
import os
import sys


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="prelude-amd", description="Qwen3 generation on one MI355X")
    ap.add_argument("--model", help="model folder (config.json + safetensors); with --random-weights, a config.json "
                                    "or a folder holding one")
    ap.add_argument("--model-path", help="same as --model (the reference's flag for a local folder)")
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "f32", "bfloat16", "float32"])
    ap.add_argument("--device", default="cuda:0")
    ap.add_argument("--random-weights", action="store_true", help="draw weights from --weights-seed instead of loading them")
    ap.add_argument("--weights-seed", type=int, default=0)
    ap.add_argument("--write-model", metavar="DIR", help="with --random-weights: write the model folder (config.json, "
                                                         "model.safetensors) there and load it from there")
    ap.add_argument("--max-running-requests", type=int, default=256)
    ap.add_argument("--max-num-batched-tokens", type=int, default=8192)
    ap.add_argument("--long-prefill-token-threshold", type=int, default=0)
    ap.add_argument("--max-total-tokens", type=int, default=0)
    ap.add_argument("--decode-reservation-cap", type=int, default=0)
    ap.add_argument("--decode-priority-max-remaining-tokens", type=int, default=4)
    ap.add_argument("--gpu-memory-utilization", type=float, default=0.9)
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--max-cache-tokens", type=int, default=None, help="tokens the cache holds (default: from free memory)")
    g = ap.add_mutually_exclusive_group()
    g.add_argument("--cuda-graph", "--hip-graph", dest="hip_graph", action="store_true", default=True)
    g.add_argument("--no-cuda-graph", "--no-hip-graph", dest="hip_graph", action="store_false")
    ap.add_argument("--hip-graph-portion-tokens", type=int, default=1024,
                    help="small steps with prompt portions are replayed from graphs up to this many tokens (0: never)")
    ap.add_argument("--no-weight-tiles", dest="weight_tiles", action="store_false", default=True,
                    help="keep no second, tiled copy of the weights for decode steps (saves their memory)")
    ap.add_argument("--no-overlap-steps", dest="overlap_steps", action="store_false", default=True,
                    help="wait for every step's token ids before scheduling the next step")
    # the request
    ap.add_argument("--prompt", action="append", default=[], help="text prompt (needs tokenizer.json); repeatable")
    ap.add_argument("--prompt-ids", action="append", default=[], help="comma-separated token ids; repeatable")
    ap.add_argument("--prompt-len", type=int, action="append", default=[],
                    help="a prompt of this many random token ids; repeatable")
    ap.add_argument("--max-tokens", type=int, default=4096)
    ap.add_argument("--temperature", type=float, default=0.7)
    ap.add_argument("--top-p", type=float, default=1.0)
    ap.add_argument("--top-k", type=int, default=None)
    ap.add_argument("--seed", type=int, default=None)
    ap.add_argument("--stop-token-ids", default="", help="comma-separated token ids that end a request")
    ap.add_argument("--logprobs", type=int, default=None, help="with every token its log-probability and the K likeliest")
    ap.add_argument("--prompt-logprobs", action="store_true", help="the log-probability of every prompt token too")
    ap.add_argument("--stop", action="append", default=[], help="a string that ends a request (needs tokenizer.json); "
                                                                 "repeatable")
    return ap


def _dtype(s: str) -> str:
    return {"bf16": "bfloat16", "f32": "float32"}.get(s, s)


def main(argv=None) -> int:
    args = build_parser().parse_args(argv)
    model = args.model_path or args.model
    if not model:
        print("error: --model is required", file=sys.stderr)
        return 2
    import numpy as np
    import torch
    from .config.engine_config import EngineConfig
    from .llm import LLM

    cfg = EngineConfig(dtype=_dtype(args.dtype), device=args.device, page_size=args.page_size,
                       max_cache_tokens=args.max_cache_tokens, gpu_memory_utilization=args.gpu_memory_utilization,
                       max_num_batched_tokens=args.max_num_batched_tokens,
                       long_prefill_token_threshold=args.long_prefill_token_threshold,
                       max_running_requests=args.max_running_requests, max_total_tokens=args.max_total_tokens,
                       decode_reservation_cap=args.decode_reservation_cap,
                       decode_priority_max_remaining_tokens=args.decode_priority_max_remaining_tokens,
                       hip_graph=args.hip_graph, hip_graph_portion_tokens=args.hip_graph_portion_tokens,
                       overlap_steps=args.overlap_steps, weight_tiles=args.weight_tiles)
    if args.random_weights:
        cfg_path = os.path.join(model, "config.json") if os.path.isdir(model) else model
        with open(cfg_path, "r", encoding="utf-8") as f:
            raw = json.load(f)
        if args.write_model:
            from .weights.random_init import write_random_model
            dt = torch.float32 if _dtype(args.dtype) == "float32" else torch.bfloat16
            print(f"writing random weights (seed {args.weights_seed}) to {args.write_model}", file=sys.stderr, flush=True)
            llm = LLM(write_random_model(raw, args.write_model, seed=args.weights_seed, dtype=dt), config=cfg)
        else:
            llm = LLM.from_config(raw, config=cfg, seed=args.weights_seed)
    else:
        llm = LLM(model, config=cfg)
    prompts = list(args.prompt)
    prompts += [[int(x) for x in s.split(",") if x.strip()] for s in args.prompt_ids]
    rng = np.random.default_rng(0 if args.seed is None else args.seed)
    prompts += [rng.integers(0, llm.engine.vocab_size, size=n).tolist() for n in args.prompt_len]
    if not prompts:
        print("error: give --prompt, --prompt-ids or --prompt-len", file=sys.stderr)
        return 2
    stop = [int(x) for x in args.stop_token_ids.split(",") if x.strip()]
    outs = llm.generate(prompts, max_tokens=args.max_tokens, temperature=args.temperature, top_p=args.top_p,
                        top_k=args.top_k, seed=args.seed, stop_token_ids=stop, stop=args.stop, logprobs=args.logprobs,
                        prompt_logprobs=args.prompt_logprobs)
    for o in outs:
        rec = {"request_id": o.request_id, "token_ids": o.token_ids, "finish_reason": o.finish_reason,
               "usage": o.usage, "metrics": {k: round(v, 3) for k, v in o.metrics.items()}}
        if o.error is not None:
            rec["error"] = o.error
        if o.text is not None:
            rec["text"] = o.text
        for key in ("token_logprobs", "top_logprobs", "prompt_logprobs"):
            if getattr(o, key) is not None:
                rec[key] = getattr(o, key)
        dec = max(o.metrics.get("decode_ms", 0.0), 1e-9)
        rec["decode_tok_per_s"] = round(max(len(o.token_ids) - 1, 0) / dec * 1e3, 1)
        print(json.dumps(rec), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
