"""The Python entry point: ``LLM(model_dir).generate(prompts, ...)``, and ``LLM.session()`` for requests that
arrive while others run.

Modelled on the reference's ``InferenceEngine::generate`` / ``generate_batch``
(crates/prelude-core/src/engine/mod.rs:75-132) and its request and result
types (crates/prelude-core/src/types.rs:388-455): per request a prompt (text
or token ids), ``max_tokens``, sampling options, stop token ids and a seed;
per result the generated ids, why it finished (``stop`` | ``length`` | ``eos`` |
``cancelled``, crates/prelude-core/src/scheduler/state.rs:35-52; ``error`` for a
request whose step failed), token counts and the four timings ``ttft_ms, prefill_ms, decode_ms, total_ms``.
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
import numbers
import os
import time
from typing import Dict, Iterable, List, Optional, Sequence, Union

import torch

from .config.engine_config import EngineConfig
from .engine.engine import Engine, StepEntry
from .engine.scheduler import Scheduler, SchedulerError
from .ops import kernels as K
from .sampling.sampler import RequestSampler, SamplingParams, sample_rows_device

DEFAULT_MAX_TOKENS = 4096   # crates/prelude-server/src/routes/generation_common.rs:9
PROMPT_LOGPROBS_CHUNK = 512

Prompt = Union[str, Sequence[int]]


@dataclasses.dataclass
class GenerationResult:
    request_id: int
    prompt_token_ids: List[int]
    token_ids: List[int]
    finish_reason: str                      # "stop" | "length" | "eos" | "cancelled" | "error"
    text: Optional[str] = None              # when a tokenizer is at hand
    error: Optional[str] = None             # with "error": what failed in the step that ended the request
    metrics: Dict[str, float] = dataclasses.field(default_factory=dict)
    preemptions: int = 0
    # asked for with ``logprobs`` / ``prompt_logprobs`` (crates/prelude-core/src/types.rs:388-455):
    token_logprobs: Optional[List[float]] = None                  # log P of each generated token
    top_logprobs: Optional[List[List[tuple]]] = None              # per generated token the k likeliest (id, log P)
    prompt_logprobs: Optional[List[Optional[float]]] = None       # log P of each prompt token given those before it

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
    logprobs: Optional[int] = None       # None: not asked for; k >= 0: the token's own and the k likeliest
    token_lps: List[float] = dataclasses.field(default_factory=list)
    top_lps: List[List[tuple]] = dataclasses.field(default_factory=list)
    prompt_lps: Optional[List[Optional[float]]] = None
    t_first: Optional[float] = None
    finish_reason: Optional[str] = None
    pending_row: Optional[int] = None    # the last of ``tokens`` is still on the device: its row among the step's samples
    done: bool = False
    preemptions: int = 0
    error: Optional[str] = None


@dataclasses.dataclass
class _InFlight:
    """A launched step whose sampled ids the host has not read yet."""
    drawn: List[_Live]
    sampled: torch.Tensor        # int32 [len(drawn)] on the device
    host: torch.Tensor           # pinned copy of it, valid once ``ready`` has passed
    ready: torch.cuda.Event
    # log-probabilities asked for, as pinned copies: of the drawn tokens (with the candidates for the k likeliest),
    # and of prompt tokens, ``prompt_at`` saying whose and where
    lp: Optional[torch.Tensor] = None
    top: Optional[tuple] = None
    prompt_lp: Optional[torch.Tensor] = None
    prompt_at: Optional[List[tuple]] = None


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
    def from_config(cls, raw_config: dict, dtype: str = "bfloat16", config: Optional[EngineConfig] = None,
                    seed: int = 0, std: float = 0.02, norm_std: float = 0.01, **overrides) -> "LLM":
        """The random-weights mode: the model ``raw_config`` (a config.json's content) describes, every tensor
        drawn on the device from (seed, tensor name); no folder is read or written."""
        cfg = config or EngineConfig()
        cfg.dtype = dtype if config is None else cfg.dtype
        for k, v in overrides.items():
            if not hasattr(cfg, k):
                raise TypeError(f"unknown engine option {k!r}")
            setattr(cfg, k, v)
        return cls.from_engine(Engine.from_config(raw_config, cfg, seed, std, norm_std))

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
                 stop: Iterable[str] = (), logprobs: Optional[int] = None,
                 prompt_logprobs: bool = False, on_token=None) -> List[GenerationResult]:
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

        ``logprobs`` = k >= 0 returns with every generated token its log-probability
        under softmax of the raw logits and the k likeliest tokens with theirs
        (postprocess.rs:88-155); ``prompt_logprobs`` the log-probability of every
        prompt token but the first given those before it (the head then runs over
        all prompt positions, not only the last).

        ``on_token(prompt_index, token_id)`` is called for every generated token as
        soon as the host has read it (the reference streams text deltas the same
        way, crates/prelude-core/src/engine/run/ar.rs:1557), in the order the
        tokens of a request are generated.
        """
        single = isinstance(prompts, str) or (len(prompts) > 0 and isinstance(prompts[0], numbers.Integral))
        plist = [prompts] if single else list(prompts)
        if sampling_params is not None and len(sampling_params) != len(plist):
            raise ValueError("sampling_params must have one entry per prompt")
        session = self.session(on_token=on_token)
        for i, p in enumerate(plist):
            sp = sampling_params[i] if sampling_params is not None else SamplingParams(temperature, top_p, top_k, seed)
            try:
                session.add(p, max_tokens=max_tokens, sampling=sp, stop_token_ids=stop_token_ids, stop=stop,
                            logprobs=logprobs, prompt_logprobs=prompt_logprobs)
            except ValueError as e:
                session.abandon()
                raise ValueError(f"prompt {i}: {e}") from None
        results: List[Optional[GenerationResult]] = [None] * len(plist)
        while session.pending:
            for index, res in session.step():
                results[index] = res
        return results  # type: ignore[return-value]

    def session(self, on_token=None) -> "Session":
        """A generation loop that requests can join while others run: ``add`` a request at any time, call
        ``step`` while ``pending``; each step returns the requests that ended in it.  One session at a time."""
        return Session(self, on_token)


class Session:
    """The reference's ``ar_loop`` (crates/prelude-core/src/engine/run/ar.rs:180-396) with the request queue in
    the caller's hands: schedule, build the step, run it, sample, finish -- one step per call."""

    def __init__(self, llm: "LLM", on_token=None):
        self.llm = llm
        self.engine = llm.engine
        self.scheduler = llm.scheduler
        self._on_token = on_token
        self._live: Dict[int, _Live] = {}
        self._in_flight: Optional[_InFlight] = None
        self._added = 0
        self._ended: List[tuple] = []

    @property
    def pending(self) -> bool:
        """Whether a request is still running or a launched step has not been read."""
        return bool(self._live) or self._in_flight is not None

    def add(self, prompt: Prompt, max_tokens: int = DEFAULT_MAX_TOKENS, sampling: Optional[SamplingParams] = None,
            stop_token_ids: Iterable[int] = (), stop: Iterable[str] = (), logprobs: Optional[int] = None,
            prompt_logprobs: bool = False) -> int:
        """Queues a request; returns its index in this session (``step`` names ended requests by it)."""
        llm = self.llm
        stop_ids = frozenset(int(t) for t in stop_token_ids)
        stop_strings = tuple(x for x in ([stop] if isinstance(stop, str) else stop) if x)
        if stop_strings:
            llm.tokenizer()
        if logprobs is not None and not 0 <= int(logprobs) <= 64:
            raise ValueError(f"logprobs {logprobs} must be within 0..64")
        ids = llm._to_ids(prompt)
        if not ids:
            raise ValueError("the prompt is empty")
        bad = [t for t in ids if not 0 <= t < self.engine.vocab_size]
        if bad:
            raise ValueError(f"token id {bad[0]} is outside the vocabulary")
        # crates/prelude-core/src/engine/model_runner/generate.rs:23-26
        max_new = min(int(max_tokens), llm.max_positions - len(ids))
        if max_new < 1:
            raise ValueError(f"the prompt has {len(ids)} tokens; the model has positions for "
                             f"{llm.max_positions} and none is left to generate")
        sp = sampling if sampling is not None else SamplingParams()
        rid = llm._next_id
        llm._next_id += 1
        # every prompt position's logits are asked for with prompt_logprobs: the head then runs over portions of
        # at most PROMPT_LOGPROBS_CHUNK rows, as in crates/prelude-core/src/engine/model_runner/paged_mixed.rs:172-270
        self.scheduler.add_request(rid, len(ids), max_new, atomic=self.engine.model.atomic_prefill,
                                   max_chunk=PROMPT_LOGPROBS_CHUNK if prompt_logprobs else 0)
        index = self._added
        self._added += 1
        self._live[rid] = _Live(rid, index, ids, list(ids), max_new, RequestSampler(sp), stop_ids, time.perf_counter(),
                                stop_strings, None if logprobs is None else int(logprobs),
                                prompt_lps=[None] * len(ids) if prompt_logprobs else None)
        return index

    def abandon(self) -> None:
        """Ends every request of the session without a result and gives back what they hold."""
        if self._in_flight is not None:
            self._in_flight.ready.synchronize()
            self._in_flight = None
        for rid in list(self._live):
            self.scheduler.finish(rid)
        self._live.clear()

    def cancel(self, index: int) -> Optional[GenerationResult]:
        """Ends one request now, whatever it was doing (the reference's ``abort_request``,
        crates/prelude-core/src/engine/run/ar.rs:436-446, crates/prelude-core/src/scheduler/state.rs:357-470):
        what it holds goes back and its result, with the tokens generated so far and the reason ``cancelled``,
        is returned.  The other requests go on.  ``None`` if no live request has this index."""
        r = next((x for x in self._live.values() if x.index == index), None)
        if r is None:
            return None
        if self._in_flight is not None and any(x is r for x in self._in_flight.drawn):
            # a launched step holds a token of it that the host has not read: read it first, so that the
            # result has every token that was generated (this may end the request by itself)
            self._resolve(self._in_flight, self._live)
            self._in_flight = None
            for i, (idx, res) in enumerate(self._ended):
                if idx == index:
                    del self._ended[i]
                    return res
        return self._end_now(r, "cancelled")

    def _end_now(self, r: _Live, reason: str, error: Optional[str] = None) -> GenerationResult:
        """Takes a live request out of the scheduler and the session and makes its result."""
        if r.rid in self._live:
            r.preemptions = self.scheduler.info(r.rid).preempt_count
            self.scheduler.finish(r.rid)
            del self._live[r.rid]
        while r.tokens and r.tokens[-1] is None:      # stand-ins of tokens that were never read
            r.tokens.pop()
        r.finish_reason, r.error, r.done = reason, error, True
        return self._result(r, time.perf_counter(), r.preemptions)

    def _fail(self, rids: Sequence[int], error: BaseException) -> None:
        """A step could not be run: every request of it ends with the reason ``error`` and gives back what it
        holds (the reference's ``fail_step``, crates/prelude-core/src/engine/run/ar.rs:1647-1665); the others go on."""
        if self._in_flight is not None:     # what the step before sampled is still wanted
            self._resolve(self._in_flight, self._live)
            self._in_flight = None
        msg = f"{type(error).__name__}: {error}"
        for rid in rids:
            r = self._live.get(rid)
            if r is not None:
                self._ended.append((r.index, self._end_now(r, "error", msg)))

    def step(self) -> List[tuple]:
        """Launches the next step (if there is anything to run) and reads the one before; returns
        ``[(index, GenerationResult)]`` for the requests that ended.  A step that cannot be run ends its own
        requests with ``finish_reason == "error"`` (``error`` says why); nothing is raised for it."""
        overlap = bool(self.llm.config.overlap_steps)
        ended_before = len(self._ended)
        launched = self._launch(self._live, self._in_flight) if self._live else None
        if launched is None and self._in_flight is None:
            if self._live and len(self._ended) == ended_before:
                raise RuntimeError("the scheduler has requests but nothing to run")
            ended, self._ended = self._ended, []
            return ended
        if not overlap and launched is not None:
            self._in_flight, launched = launched, None
        if self._in_flight is not None:
            self._resolve(self._in_flight, self._live)
        self._in_flight = launched
        ended, self._ended = self._ended, []
        return ended

    @property
    def eos_token_ids(self):
        return self.llm.eos_token_ids

    @property
    def _tokenizer(self):
        return self.llm._tokenizer

    def _launch(self, live: Dict[int, _Live], previous: Optional[_InFlight]) -> Optional[_InFlight]:
        """Schedules and launches one step; the scheduler is told at once that its tokens exist."""
        try:
            portions = self.scheduler.schedule()
        except SchedulerError as e:
            # no running request can move and none can be evicted: those that run end here, the queue goes on
            self._fail([rid for rid in list(live) if self.scheduler.info(rid).running], e)
            return None
        if not portions:
            return None
        entries = []
        draw_rows: List[int] = []        # rows of the step's logits that are sampled from, in the order of `drawn`
        prompt_rows: List[int] = []      # rows whose log-probability of the next prompt token is asked for
        prompt_ids: List[int] = []
        prompt_at: List[tuple] = []
        rows = 0
        for p in portions:
            r = live[p.id]
            toks = r.tokens[p.start:p.start + p.count]
            carry = None
            if toks[-1] is None:       # sampled by the step before, not read yet
                toks = toks[:-1] + [0]
                carry = r.pending_row
            want = []
            if r.prompt_lps is not None:
                # position j says how likely prompt token j + 1 is
                for j in range(p.start, min(p.start + p.count, len(r.prompt) - 1)):
                    prompt_rows.append(rows + len(want))
                    prompt_ids.append(r.prompt[j + 1])
                    prompt_at.append((r, j + 1))
                    want.append(j - p.start)
            if p.samples:
                if not want or want[-1] != p.count - 1:
                    want.append(p.count - 1)
                draw_rows.append(rows + len(want) - 1)
            rows += len(want)
            entries.append(StepEntry(p.id, toks, want, carry))
        try:
            logits = self.engine.run(entries, [p.start for p in portions],
                                     previous.sampled if previous is not None else None)
        except Exception as e:
            self.scheduler.step_cancelled()
            self._fail([p.id for p in portions], e)
            return None
        self.scheduler.step_done()
        self.llm.steps += 1
        drawn = [live[p.id] for p in portions if p.samples]
        device = logits.device
        drawn_logits = logits
        if rows != len(draw_rows):      # other rows were asked for as well: take the sampled ones out
            drawn_logits = logits.index_select(0, torch.tensor(draw_rows, dtype=torch.int64, device=device))
        sampled = sample_rows_device(drawn_logits, [r.sampler for r in drawn])
        host = torch.empty(len(drawn), dtype=torch.int32, pin_memory=True)
        host.copy_(sampled, non_blocking=True)
        lp = top = prompt_lp = None
        ks = [r.logprobs for r in drawn if r.logprobs is not None]
        if ks:
            lp_dev, top_dev = K.logprobs(drawn_logits, sampled, max(ks))
            lp = torch.empty(lp_dev.shape, dtype=lp_dev.dtype, pin_memory=True)
            lp.copy_(lp_dev, non_blocking=True)
            if top_dev is not None:
                top = tuple(torch.empty(t.shape, dtype=t.dtype, pin_memory=True) for t in top_dev)
                for dst, src in zip(top, top_dev):
                    dst.copy_(src, non_blocking=True)
        if prompt_rows:
            sel = logits.index_select(0, torch.tensor(prompt_rows, dtype=torch.int64, device=device))
            plp_dev, _ = K.logprobs(sel, torch.tensor(prompt_ids, dtype=torch.int32, device=device))
            prompt_lp = torch.empty(plp_dev.shape, dtype=plp_dev.dtype, pin_memory=True)
            prompt_lp.copy_(plp_dev, non_blocking=True)
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
        return _InFlight(drawn, sampled, host, ready, lp, top, prompt_lp, prompt_at)

    def _resolve(self, step: _InFlight, live: Dict[int, _Live]) -> None:
        """Reads a step's sampled ids and ends the requests they end."""
        step.ready.synchronize()
        toks = step.host.tolist()
        t = time.perf_counter()
        if step.prompt_lp is not None:
            for (r, at), v in zip(step.prompt_at, step.prompt_lp.tolist()):
                r.prompt_lps[at] = v
        lps = step.lp.tolist() if step.lp is not None else None
        for row, (r, tok) in enumerate(zip(step.drawn, toks)):
            if r.done:                 # ended by an earlier token while this step was already running
                continue
            if r.logprobs is not None:
                r.token_lps.append(lps[row])
                if r.logprobs > 0:
                    vals, idx, count = step.top
                    n = int(count[row])
                    cand = sorted(zip(idx[row, :n].tolist(), vals[row, :n].tolist()), key=lambda c: (-c[1], c[0]))
                    r.top_lps.append(cand[:r.logprobs])
            at = len(r.tokens) - 1
            if at >= 1 and r.tokens[at - 1] is None:   # the step launched since then has put its own stand-in behind
                at -= 1
            r.tokens[at] = int(tok)
            if r.t_first is None:
                r.t_first = t
            if self._on_token is not None:
                self._on_token(r.index, int(tok))
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
            self._ended.append((r.index, self._result(r, t, r.preemptions)))

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
        res = GenerationResult(r.rid, list(r.prompt), out, r.finish_reason or "length", text, r.error, metrics,
                               preemptions)
        if r.logprobs is not None:
            res.token_logprobs = r.token_lps[:len(out)]
            if r.logprobs > 0:
                res.top_logprobs = r.top_lps[:len(out)]
        res.prompt_logprobs = r.prompt_lps
        return res


def generate(model: str, prompts, dtype: str = "bfloat16", **kwargs) -> List[GenerationResult]:
    """One-shot convenience: load ``model`` and generate."""
    engine_keys = {f.name for f in dataclasses.fields(EngineConfig)}
    eng = {k: kwargs.pop(k) for k in list(kwargs) if k in engine_keys and k != "dtype"}
    return LLM(model, dtype=dtype, **eng).generate(prompts, **kwargs)
