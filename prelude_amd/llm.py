"""The Python entry point: ``LLM(model_dir).generate(prompts, ...)``.

Modelled on the reference's ``InferenceEngine::generate`` / ``generate_batch``
(crates/prelude-core/src/engine/mod.rs:75-132) and its request and result
types (crates/prelude-core/src/types.rs:388-455): per request a prompt (text
or token ids), ``max_tokens``, sampling options, stop token ids and a seed;
per result the generated ids, why it finished (``stop`` | ``length`` | ``eos``),
token counts and the four timings ``ttft_ms, prefill_ms, decode_ms, total_ms``.
The loop is the reference's ``ar_loop`` (crates/prelude-core/src/engine/run/ar.rs:180-396):
schedule, build the step, run it, sample, finish.  With ``overlap_steps`` the
host runs one step ahead of the device: step N+1 is scheduled and launched
while step N still runs, taking N's sampled ids on the device, and N's ids are
read only afterwards.  What is computed, and so every token, is the same as
in the synchronous loop; a request that ends on a token's value (EOS, a stop
id) has by then been fed one step too many, whose sample is dropped.
"""
from __future__ import annotations

import dataclasses
import os
import time
from typing import Dict, Iterable, List, Optional, Sequence, Union

import torch

from .config.engine_config import EngineConfig
from .engine.engine import Engine, StepEntry
from .engine.scheduler import Scheduler
from .sampling.sampler import RequestSampler, SamplingParams, sample_rows_device

DEFAULT_MAX_TOKENS = 4096   # crates/prelude-server/src/routes/generation_common.rs:9

Prompt = Union[str, Sequence[int]]


@dataclasses.dataclass
class GenerationResult:
    request_id: int
    prompt_token_ids: List[int]
    token_ids: List[int]
    finish_reason: str                      # "stop" | "length" | "eos"
    text: Optional[str] = None              # when a tokenizer is at hand
    metrics: Dict[str, float] = dataclasses.field(default_factory=dict)
    preemptions: int = 0

    @property
    def usage(self) -> Dict[str, int]:
        n, m = len(self.prompt_token_ids), len(self.token_ids)
        return {"prompt_tokens": n, "completion_tokens": m, "total_tokens": n + m}


@dataclasses.dataclass
class _Live:
    rid: int
    index: int
    prompt: List[int]
    tokens: List[int]            # prompt + generated
    max_new: int
    sampler: RequestSampler
    stop_ids: frozenset
    t_arrive: float
    stop_strings: tuple = ()
    t_first: Optional[float] = None
    finish_reason: Optional[str] = None
    pending_row: Optional[int] = None    # the last of ``tokens`` is still on the device: its row among the step's samples
    done: bool = False
    preemptions: int = 0


@dataclasses.dataclass
class _InFlight:
    """A launched step whose sampled ids the host has not read yet."""
    drawn: List[_Live]
    sampled: torch.Tensor        # int32 [len(drawn)] on the device
    host: torch.Tensor           # pinned copy of it, valid once ``ready`` has passed
    ready: torch.cuda.Event


class LLM:
    def __init__(self, model: str, dtype: str = "bfloat16", config: Optional[EngineConfig] = None, **overrides):
        """``model``: a folder with config.json and safetensors files.  Other
        keyword arguments override fields of ``EngineConfig``."""
        cfg = config or EngineConfig()
        cfg.dtype = dtype if config is None else cfg.dtype
        for k, v in overrides.items():
            if not hasattr(cfg, k):
                raise TypeError(f"unknown engine option {k!r}")
            setattr(cfg, k, v)
        self.model_dir = model
        self._attach(Engine.from_model_dir(model, cfg))

    @classmethod
    def from_engine(cls, engine: Engine, model_dir: Optional[str] = None) -> "LLM":
        """An LLM around an engine that is already built (its ``config`` gives the scheduler's limits);
        ``model_dir`` is only needed for text prompts (its tokenizer.json)."""
        self = cls.__new__(cls)
        self.model_dir = model_dir
        self._attach(engine)
        return self

    def _attach(self, engine: Engine) -> None:
        cfg = engine.config
        self.config = cfg
        self.engine = engine
        spec = self.engine.model.spec
        self.eos_token_ids = frozenset(spec.eos_token_ids)
        self.max_positions = spec.max_positions
        cap = cfg.decode_reservation_cap or self.max_positions
        self.scheduler = Scheduler(self.engine.tables, cfg.max_num_batched_tokens, cfg.long_prefill_token_threshold,
                                   cfg.max_running_requests, cfg.max_total_tokens, cap,
                                   cfg.decode_priority_max_remaining_tokens, self.engine.model.needs_state)
        self._next_id = 0
        self._tokenizer = None
        self.steps = 0

    # ---- tokenizer (only when prompts are text) --------------------------------
    def tokenizer(self):
        if self._tokenizer is None:
            path = os.path.join(self.model_dir or "", "tokenizer.json")
            if not os.path.isfile(path):
                raise ValueError(f"text prompts need {path}; pass token ids instead")
            from tokenizers import Tokenizer
            self._tokenizer = Tokenizer.from_file(path)
        return self._tokenizer

    def _to_ids(self, prompt: Prompt) -> List[int]:
        if isinstance(prompt, str):
            return list(self.tokenizer().encode(prompt).ids)
        return [int(t) for t in prompt]

    # ---- generation -----------------------------------------------------------------
    def generate(self, prompts: Union[Prompt, Sequence[Prompt]], max_tokens: int = DEFAULT_MAX_TOKENS,
                 temperature: float = 0.7, top_p: float = 1.0, top_k: Optional[int] = None,
                 seed: Optional[int] = None, stop_token_ids: Iterable[int] = (),
                 sampling_params: Optional[Sequence[SamplingParams]] = None,
                 stop: Iterable[str] = ()) -> List[GenerationResult]:
        """Runs all prompts to their end with continuous batching; results in the order of the prompts.

        ``sampling_params`` gives each prompt options of its own and overrides
        temperature/top_p/top_k/seed.  A request ends on an EOS id of the
        model (``eos``), on one of ``stop_token_ids`` (``stop``), after
        ``max_tokens`` tokens, clamped to the positions the model has left (``length``),
        or once its text holds one of the strings ``stop`` (``stop``; needs the
        folder's tokenizer.json; the text returned ends before the string, the
        token ids keep the tokens that spelt it:
        crates/prelude-core/src/engine/run/ar.rs:1560-1577,
        crates/prelude-core/src/engine/model_runner/postprocess.rs:5-16).
        """
        single = isinstance(prompts, str) or (len(prompts) > 0 and isinstance(prompts[0], int))
        plist = [prompts] if single else list(prompts)
        if sampling_params is not None and len(sampling_params) != len(plist):
            raise ValueError("sampling_params must have one entry per prompt")
        stop_ids = frozenset(int(t) for t in stop_token_ids)
        stop_strings = tuple(s for s in ([stop] if isinstance(stop, str) else stop) if s)
        if stop_strings:
            self.tokenizer()
        live: Dict[int, _Live] = {}
        results: List[Optional[GenerationResult]] = [None] * len(plist)
        now = time.perf_counter()
        for i, p in enumerate(plist):
            ids = self._to_ids(p)
            if not ids:
                raise ValueError(f"prompt {i} is empty")
            bad = [t for t in ids if not 0 <= t < self.engine.vocab_size]
            if bad:
                raise ValueError(f"prompt {i}: token id {bad[0]} is outside the vocabulary")
            # crates/prelude-core/src/engine/model_runner/generate.rs:23-26
            max_new = min(int(max_tokens), self.max_positions - len(ids))
            if max_new < 1:
                raise ValueError(f"prompt {i} has {len(ids)} tokens; the model has positions for "
                                 f"{self.max_positions} and none is left to generate")
            sp = sampling_params[i] if sampling_params is not None else SamplingParams(temperature, top_p, top_k, seed)
            rid = self._next_id
            self._next_id += 1
            self.scheduler.add_request(rid, len(ids), max_new)
            live[rid] = _Live(rid, i, ids, list(ids), max_new, RequestSampler(sp), stop_ids, now, stop_strings)

        overlap = bool(self.config.overlap_steps)
        in_flight: Optional[_InFlight] = None
        while live or in_flight is not None:
            launched = self._launch(live, in_flight) if live else None
            if launched is None and in_flight is None:
                raise RuntimeError("the scheduler has requests but nothing to run")
            if not overlap and launched is not None:
                in_flight, launched = launched, None
            if in_flight is not None:
                self._resolve(in_flight, live, results)
            in_flight = launched
        return results  # type: ignore[return-value]

    def _launch(self, live: Dict[int, _Live], previous: Optional[_InFlight]) -> Optional[_InFlight]:
        """Schedules and launches one step; the scheduler is told at once that its tokens exist."""
        portions = self.scheduler.schedule()
        if not portions:
            return None
        entries = []
        for p in portions:
            r = live[p.id]
            toks = r.tokens[p.start:p.start + p.count]
            carry = None
            if toks[-1] is None:       # sampled by the step before, not read yet
                toks = toks[:-1] + [0]
                carry = r.pending_row
            entries.append(StepEntry(p.id, toks, [p.count - 1] if p.samples else [], carry))
        try:
            logits = self.engine.run(entries, [p.start for p in portions],
                                     previous.sampled if previous is not None else None)
        except Exception:
            self.scheduler.step_cancelled()
            raise
        self.scheduler.step_done()
        self.steps += 1
        drawn = [live[p.id] for p in portions if p.samples]
        sampled = sample_rows_device(logits, [r.sampler for r in drawn])
        host = torch.empty(len(drawn), dtype=torch.int32, pin_memory=True)
        host.copy_(sampled, non_blocking=True)
        ready = torch.cuda.Event()
        ready.record()
        for row, r in enumerate(drawn):
            self.scheduler.on_token(r.rid)
            r.tokens.append(None)
            r.pending_row = row
            if len(r.tokens) - len(r.prompt) >= r.max_new:
                # the last token it may have, whatever its value: nothing more is scheduled for it
                r.preemptions = self.scheduler.info(r.rid).preempt_count
                self.scheduler.finish(r.rid)
                r.finish_reason = "length"
                del live[r.rid]
        return _InFlight(drawn, sampled, host, ready)

    def _resolve(self, step: _InFlight, live: Dict[int, _Live], results: List[Optional[GenerationResult]]) -> None:
        """Reads a step's sampled ids and ends the requests they end."""
        step.ready.synchronize()
        toks = step.host.tolist()
        t = time.perf_counter()
        for r, tok in zip(step.drawn, toks):
            if r.done:                 # ended by an earlier token while this step was already running
                continue
            at = len(r.tokens) - 1
            if at >= 1 and r.tokens[at - 1] is None:   # the step launched since then has put its own stand-in behind
                at -= 1
            r.tokens[at] = int(tok)
            if r.t_first is None:
                r.t_first = t
            # order of checks: crates/prelude-core/src/engine/run/ar.rs:1525-1578
            if tok in self.eos_token_ids:
                reason = "eos"
            elif tok in r.stop_ids:
                reason = "stop"
            elif at + 1 - len(r.prompt) >= r.max_new:
                reason = "length"
            elif r.stop_strings and self._holds_stop_string(r, at):
                reason = "stop"
            else:
                continue
            del r.tokens[at + 1:]
            if r.rid in live:          # ended by the token's value: the scheduler still holds it
                r.preemptions = self.scheduler.info(r.rid).preempt_count
                self.scheduler.finish(r.rid)
                del live[r.rid]
            r.finish_reason = reason
            r.done = True
            results[r.index] = self._result(r, t, r.preemptions)

    def _holds_stop_string(self, r: _Live, at: int) -> bool:
        text = self._tokenizer.decode(r.tokens[len(r.prompt):at + 1])
        return any(s in text for s in r.stop_strings)

    def _result(self, r: _Live, t_end: float, preemptions: int) -> GenerationResult:
        out = r.tokens[len(r.prompt):]
        first = r.t_first if r.t_first is not None else t_end
        metrics = {"ttft_ms": (first - r.t_arrive) * 1e3, "prefill_ms": (first - r.t_arrive) * 1e3,
                   "decode_ms": (t_end - first) * 1e3, "total_ms": (t_end - r.t_arrive) * 1e3}
        text = None
        if self._tokenizer is not None:
            text = self._tokenizer.decode(out)
            for s in r.stop_strings:      # cut at the first occurrence of each, in the order given
                cut = text.find(s)
                if cut >= 0:
                    text = text[:cut]
        return GenerationResult(r.rid, list(r.prompt), out, r.finish_reason or "length", text, metrics, preemptions)


def generate(model: str, prompts, dtype: str = "bfloat16", **kwargs) -> List[GenerationResult]:
    """One-shot convenience: load ``model`` and generate."""
    engine_keys = {f.name for f in dataclasses.fields(EngineConfig)}
    eng = {k: kwargs.pop(k) for k in list(kwargs) if k in engine_keys and k != "dtype"}
    return LLM(model, dtype=dtype, **eng).generate(prompts, **kwargs)
