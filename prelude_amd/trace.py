"""Trace replay: drives the engine's own step function with given tokens.

It owns no forward pass, cache or loader: ``TraceRunner`` is a thin loop over
``Engine.step`` and ``Engine.release``.  Request ids of any JSON type are
mapped to the engine's integer ids.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence

import numpy as np
import torch

from .config.engine_config import EngineConfig
from .engine.engine import Engine, StepEntry


class TraceRunner:
    def __init__(self, model_dir: str, dtype: str, max_tokens: int, page_size: Optional[int] = None,
                 device: str = "cuda:0"):
        cfg = EngineConfig(dtype=dtype, device=device)
        if page_size is not None:
            cfg.page_size = page_size
        # the pool holds exactly what live requests may hold, so pages are used again
        cfg.max_cache_tokens = max(int(max_tokens), cfg.page_size)
        self.engine = Engine.from_model_dir(model_dir, cfg)
        self._ids: Dict[object, int] = {}
        self._next = 0

    def _rid(self, key) -> int:
        key = key if isinstance(key, (str, int)) else repr(key)
        if key not in self._ids:
            self._ids[key] = self._next
            self._next += 1
        return self._ids[key]

    def step(self, entries: Sequence[dict], end: Sequence[object] = ()) -> Optional[np.ndarray]:
        """Runs one step; returns the wanted logits [wanted, vocab] as float32, or None if none were wanted."""
        out = None
        if entries:
            batch = [StepEntry(self._rid(e["id"]), list(e["tokens"]), list(e.get("want", []))) for e in entries]
            logits = self.engine.step(batch)
            if logits.shape[0] > 0:
                out = logits.to(torch.float32).cpu().numpy()
            else:
                torch.cuda.synchronize()
        for key in end:
            key = key if isinstance(key, (str, int)) else repr(key)
            if key in self._ids:
                self.engine.release(self._ids.pop(key))
        return out
