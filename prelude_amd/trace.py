"""Trace replay: drives the engine's own step function with given tokens.

It owns no forward pass, cache or loader: ``TraceRunner`` is a thin loop over
``Engine.step`` and ``Engine.release``.  Request ids of any JSON type are
mapped to the engine's integer ids.
"""
from __future__ import annotations

from typing import Dict, Optional, Sequence

import numpy as np
import torch

from .config.engine_config import EngineConfig
from .engine.engine import Engine, StepEntry


class TraceRunner:
    def __init__(self, model_dir: Optional[str], dtype: str, max_tokens: Optional[int] = None,
                 page_size: Optional[int] = None, device: str = "cuda:0", num_pages: Optional[int] = None,
                 random_config: Optional[dict] = None, weights_seed: int = 0):
        """``model_dir``: a folder with config.json and safetensors; or ``random_config`` (a config.json's
        content): that model with weights drawn on the device from ``weights_seed``.  The pool holds
        ``max_tokens`` tokens, or ``num_pages`` pages of ``page_size`` tokens: exactly what live requests may
        hold, so pages are used again."""
        cfg = EngineConfig(dtype=dtype, device=device)
        if page_size is not None:
            cfg.page_size = int(page_size)
        if num_pages is not None:
            tokens = int(num_pages) * cfg.page_size
        elif max_tokens is not None:
            tokens = int(max_tokens)
        else:
            raise ValueError("trace replay needs the pool's size: max_tokens or num_pages")
        cfg.max_cache_tokens = max(tokens, cfg.page_size)
        # a step may bring as much as the pool holds (a whole request at once)
        cfg.max_num_batched_tokens = max(cfg.max_num_batched_tokens, cfg.max_cache_tokens)
        if random_config is not None:
            self.engine = Engine.from_config(random_config, cfg, seed=weights_seed)
        else:
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
