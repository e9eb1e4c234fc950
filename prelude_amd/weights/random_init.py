"""The random-weights mode, in two forms: a model folder (config.json,
model.safetensors) written from a configuration and a seed, and the same
draw made straight on the device for models too large to write out first.

The reference has no such mode (its nearest is all-zero weights,
crates/prelude-core/src/engine/weight_loader.rs:317-333).  Every tensor is
drawn from (seed, tensor name), so a tensor's values do not depend on which
other tensors the model has: matrices and biases N(0, std), norm scales
1 + N(0, norm_std).

One generator serves both forms, and it gives the same values on the CPU and
on the GPU, bit for bit: a seed names one model, whether it is written to a
folder or drawn into device memory.  An element's value follows from its
index alone: three words of a counter-based hash (the splitmix64 finalizer
over seed + index, in wrapping 64-bit integer arithmetic, which every device
computes alike) are cut into twelve 16-bit fields whose sum, centred and
scaled, is normal to well past four deviations (the sum of twelve uniform
numbers; it cannot exceed six).  The only floating-point steps are an exact
conversion of that small integer, one multiplication and, for norm scales,
one addition: no library function whose last bit could differ between
devices.
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


_GAMMA = 0x9E3779B97F4A7C15 - (1 << 64)      # the hash's constants as signed 64-bit numbers
_MUL1 = 0xBF58476D1CE4E5B9 - (1 << 64)
_MUL2 = 0x94D049BB133111EB - (1 << 64)
_CHUNK = 1 << 24                              # elements drawn at a time (bounds the temporaries: some 1 GB)


def _mix(z: torch.Tensor) -> torch.Tensor:
    """The splitmix64 finalizer on int64 tensors; shifts are made logical by masking the sign's copies away."""
    z = (z ^ ((z >> 30) & 0x3FFFFFFFF)) * _MUL1
    z = (z ^ ((z >> 27) & 0x1FFFFFFFFF)) * _MUL2
    return z ^ ((z >> 31) & 0x1FFFFFFFF)


def _standard_normal(n: int, key: int, device: torch.device) -> torch.Tensor:
    """n draws of N(0, 1) as float32, element i from (key, i) alone; the same bits on every device."""
    out = torch.empty(n, dtype=torch.float32, device=device)
    for lo in range(0, n, _CHUNK):
        hi = min(n, lo + _CHUNK)
        idx = torch.arange(lo, hi, dtype=torch.int64, device=device) * 3
        total = torch.zeros(hi - lo, dtype=torch.int64, device=device)
        for word in range(3):
            z = _mix((idx + word) * _GAMMA + key)
            for shift in (0, 16, 32, 48):
                total += (z >> shift) & 0xFFFF
        # twelve fields of mean 32767.5 and variance (2^32 - 1) / 12 each
        out[lo:hi] = (total - 393210).to(torch.float32) * (1.0 / 65536.0)
    return out


def _draw(name: str, req, seed: int, std: float, norm_std: float, device: torch.device) -> torch.Tensor:
    n = 1
    for d in req.shape:
        n *= int(d)
    t = _standard_normal(n, _seed_for(seed, name), device).reshape(req.shape)
    # one multiplication, then (for norm scales) one addition: separate steps, so no device contracts them
    return t.mul_(norm_std).add_(1.0) if req.kind == NORM else t.mul_(std)


def random_tensors(raw_config: Mapping[str, Any], seed: int, std: float = 0.02, norm_std: float = 0.01,
                   dtype: torch.dtype = torch.bfloat16, device=None) -> dict:
    """Every tensor of the architecture ``raw_config`` names, by checkpoint name, on the CPU: all of them rounded
    to ``dtype``.  Drawn on ``device`` (the GPU when there is one: the values are the same, the draw is faster)."""
    from ..models.causal_lm import CausalLM
    arch = resolve_architecture(raw_config)
    model = CausalLM(arch.build_spec(arch.parse_config(raw_config)))
    if device is None:
        device = "cuda" if torch.cuda.is_available() else "cpu"
    device = torch.device(device)
    return {name: _draw(name, req, seed, std, norm_std, device).to(dtype).cpu()
            for name, req in model.tensor_requests().items()}


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


def load_random(model, dtype: torch.dtype, device: torch.device, seed: int = 0, std: float = 0.02,
                norm_std: float = 0.01) -> None:
    """Loads ``model`` (a ``CausalLM``) with tensors drawn on ``device``: what ``load_into`` does for a folder,
    without one.  Nothing the size of the model exists on the host or on disk at any time."""
    cache = {}

    def fetch(name: str, req):
        want = dtype if req.kind == MATRIX else torch.float32
        key = (name, want)
        if key not in cache:      # a tensor named twice (a tied head) is drawn once and shared
            cache[key] = _draw(name, req, seed, std, norm_std, device).to(want).contiguous()
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
    return {name: _draw(name, req, seed, std, norm_std, device).to(dtype if req.kind == MATRIX else torch.float32)
            for name, req in model.tensor_requests().items()}
