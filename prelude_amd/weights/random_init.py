"""The random-weights mode, in two forms: a model folder (config.json,
model.safetensors) written from a configuration and a seed, and the same
draw made straight on the device for models too large to write out first.

The reference has no such mode (its nearest is all-zero weights,
crates/prelude-core/src/engine/weight_loader.rs:317-333).  Every tensor is
drawn from a generator seeded by (seed, tensor name), so a tensor's values do
not depend on which other tensors the model has: matrices and biases
N(0, std), norm scales 1 + N(0, norm_std).  The folder is drawn with the
CPU's generator and the device form with the GPU's: the same seed gives the
same distribution and other values.
"""
from __future__ import annotations

import hashlib
import json
import os
from typing import Any, Mapping

import torch

from ..config.registry import resolve_architecture
from ..parts.base import MATRIX, NORM
from .safetensors_io import write_safetensors


def _seed_for(seed: int, name: str) -> int:
    h = hashlib.sha256(f"{seed}:{name}".encode()).digest()
    return int.from_bytes(h[:8], "little") & 0x7FFFFFFFFFFFFFFF


def random_tensors(raw_config: Mapping[str, Any], seed: int, std: float = 0.02, norm_std: float = 0.01,
                   dtype: torch.dtype = torch.bfloat16) -> dict:
    from ..models.causal_lm import CausalLM
    arch = resolve_architecture(raw_config)
    model = CausalLM(arch.build_spec(arch.parse_config(raw_config)))
    out = {}
    for name, req in model.tensor_requests().items():
        g = torch.Generator().manual_seed(_seed_for(seed, name))
        t = torch.randn(req.shape, generator=g, dtype=torch.float32)
        t = 1.0 + norm_std * t if req.kind == NORM else std * t
        out[name] = t.to(dtype)
    return out


def write_random_model(raw_config: Mapping[str, Any], out_dir: str, seed: int = 0, std: float = 0.02,
                       norm_std: float = 0.01, dtype: torch.dtype = torch.bfloat16) -> str:
    """Writes ``out_dir/config.json`` and ``out_dir/model.safetensors``; returns ``out_dir``."""
    tensors = random_tensors(raw_config, seed, std, norm_std, dtype)
    os.makedirs(out_dir, exist_ok=True)
    with open(os.path.join(out_dir, "config.json"), "w", encoding="utf-8") as f:
        json.dump(dict(raw_config), f, indent=1)
    write_safetensors(os.path.join(out_dir, "model.safetensors"), tensors,
                      {"format": "pt", "seed": str(seed), "std": str(std), "norm_std": str(norm_std)})
    return out_dir


def _draw_on_device(name: str, req, seed: int, std: float, norm_std: float, device: torch.device) -> torch.Tensor:
    g = torch.Generator(device=device).manual_seed(_seed_for(seed, name))
    t = torch.randn(req.shape, generator=g, device=device, dtype=torch.float32)
    return t.mul_(norm_std).add_(1.0) if req.kind == NORM else t.mul_(std)


def load_random(model, dtype: torch.dtype, device: torch.device, seed: int = 0, std: float = 0.02,
                norm_std: float = 0.01) -> None:
    """Loads ``model`` (a ``CausalLM``) with tensors drawn on ``device``: what ``load_into`` does for a folder,
    without one.  Nothing the size of the model exists on the host or on disk at any time."""
    cache = {}

    def fetch(name: str, req):
        want = dtype if req.kind == MATRIX else torch.float32
        key = (name, want)
        if key not in cache:      # a tensor named twice (a tied head) is drawn once and shared
            cache[key] = _draw_on_device(name, req, seed, std, norm_std, device).to(want).contiguous()
        return cache[key]

    model.load(fetch, dtype, device)


def random_tensors_on_device(raw_config: Mapping[str, Any], seed: int, device, std: float = 0.02,
                             norm_std: float = 0.01, dtype: torch.dtype = torch.bfloat16) -> dict:
    """The tensors ``load_random`` gives a model of this configuration, by checkpoint name (matrices rounded to
    ``dtype``, the others 32-bit): for writing them out or comparing against them."""
    from ..models.causal_lm import CausalLM
    arch = resolve_architecture(raw_config)
    model = CausalLM(arch.build_spec(arch.parse_config(raw_config)))
    device = torch.device(device)
    return {name: _draw_on_device(name, req, seed, std, norm_std, device).to(dtype if req.kind == MATRIX else torch.float32)
            for name, req in model.tensor_requests().items()}
