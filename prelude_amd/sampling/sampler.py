"""From logits rows to token ids: greedy, temperature, top-k, top-p, seeded per request.

Which mode a request gets follows
crates/prelude-core/src/engine/model_runner/postprocess.rs:18-37: temperature
below 1e-7 is greedy; else top_k > 0 selects top-k then top-p, else top_p < 1
selects top-p, else the whole distribution.  One random number is consumed per
generated token from a generator seeded per request (default seed 42,
crates/prelude-core/src/constants.rs:4).  The draw itself happens on the device
(``csrc/kernels/sampling.hip``); the generator is numpy's Philox, not the
reference's, so the same seed gives other tokens than the reference would.
"""
from __future__ import annotations

import dataclasses
from typing import List, Optional, Sequence

import numpy as np
import torch

from ..ops import kernels as K

DEFAULT_SEED = 42
GREEDY_BELOW = 1e-7


@dataclasses.dataclass
class SamplingParams:
    temperature: float = 0.7       # the reference's API default (crates/prelude-server/src/routes/generation_common.rs:54-55)
    top_p: float = 1.0
    top_k: Optional[int] = None
    seed: Optional[int] = None

    def validate(self) -> None:
        if not (self.temperature >= 0.0):
            raise ValueError(f"temperature {self.temperature} must be >= 0")
        if not (0.0 <= self.top_p <= 1.0):
            raise ValueError(f"top_p {self.top_p} must be within [0, 1]")
        if self.top_k is not None and self.top_k < 0:
            raise ValueError(f"top_k {self.top_k} must be >= 0")

    @property
    def greedy(self) -> bool:
        return self.temperature < GREEDY_BELOW


class RequestSampler:
    """A request's sampling state: its parameters and its random stream."""

    def __init__(self, params: SamplingParams):
        params.validate()
        self.params = params
        seed = DEFAULT_SEED if params.seed is None else int(params.seed)
        self._rng = np.random.Generator(np.random.Philox(seed))

    def next_uniform(self) -> float:
        return float(self._rng.random(dtype=np.float32))


def sample_rows_device(logits: torch.Tensor, samplers: Sequence[RequestSampler]) -> torch.Tensor:
    """One token id per row of float32 logits [R, V], left on the device as int32 [R]; row i belongs to samplers[i].

    Nothing here waits for the device: the ids can feed the next step where
    they are (``Engine.step(..., carried=ids)``) and be read by the host later.
    """
    r = logits.shape[0]
    if r != len(samplers):
        raise ValueError(f"{r} logits rows for {len(samplers)} requests")
    if r == 0:
        return torch.empty(0, dtype=torch.int32, device=logits.device)
    if all(s.params.greedy for s in samplers):
        return K.argmax(logits)
    host = torch.empty((3, r), dtype=torch.float32, pin_memory=True)
    topk = torch.zeros(r, dtype=torch.int32, pin_memory=True)
    hv, kv = host.numpy(), topk.numpy()
    for i, s in enumerate(samplers):
        p = s.params
        hv[0, i] = 0.0 if p.greedy else p.temperature
        # top_p outside (0, 1) keeps everything (crates/prelude-core/src/engine/sampling/logits_processor.rs:119-125)
        hv[1, i] = p.top_p
        hv[2, i] = 0.0 if p.greedy else s.next_uniform()
        kv[i] = p.top_k or 0
    dev = host.to(logits.device, non_blocking=True)
    dk = topk.to(logits.device, non_blocking=True)
    return K.sample(logits, dev[0], dk, dev[1], dev[2],
                    any_top_k=any((s.params.top_k or 0) > 0 for s in samplers if not s.params.greedy),
                    any_top_p=any(0.0 < s.params.top_p < 1.0 for s in samplers if not s.params.greedy))


def sample_rows(logits: torch.Tensor, samplers: Sequence[RequestSampler]) -> List[int]:
    """As ``sample_rows_device``, read back: waits for the device."""
    return sample_rows_device(logits, samplers).tolist()
