"""Brings a model's tensors from safetensors files to the device, by name.

What the reference does per tensor (fetch by dotted name, cast to the engine's
type, then check the shape: crates/prelude-core/src/engine/weight_loader.rs:200-285,
:379-404) is done here for the whole model at once, before anything is copied:
one error lists every missing tensor, every unexpected one and every wrong shape.
The reference passes over whatever it does not fetch; here only the names an
architecture declares it may meet and does not read (``ModelSpec.ignored_tensors``:
the unused head of a tied checkpoint, exported rotary frequencies) are passed
over, and anything else nothing asks for is reported, since it most often
means the wrong architecture or a renamed tensor.

Element types on the device: matrices take the engine's type (bfloat16 for
serving, float32 for the 32-bit path); norm scales and biases are always
float32, so a tensor stored in 32-bit stays so and a bfloat16 one is widened
exactly; integer tensors become int32.
"""
from __future__ import annotations

import fnmatch
from typing import Dict, Mapping, Sequence, Tuple

import torch

from ..parts.base import MATRIX, TensorReq
from .safetensors_io import WeightFiles


class WeightError(ValueError):
    pass


def check_tensors(requests: Mapping[str, TensorReq], files: WeightFiles, where: str,
                  ignored: Sequence[str] = ()) -> None:
    """``ignored``: shell patterns of names the files may hold although nothing asks for them."""
    missing, wrong = [], []
    for name, req in requests.items():
        if name not in files:
            missing.append(name)
            continue
        dt, shape = files.info(name)
        if tuple(shape) != tuple(req.shape):
            wrong.append(f"{name}: expected {list(req.shape)}, got {list(shape)}")
        elif not (dt.is_floating_point or dt in (torch.int32, torch.int64)):
            wrong.append(f"{name}: element type {dt} cannot be used")
    unexpected = [n for n in files.names() if n not in requests and not any(fnmatch.fnmatchcase(n, p) for p in ignored)]
    if missing or wrong or unexpected:
        def part(title, items):
            if not items:
                return ""
            shown = "\n    ".join(sorted(items)[:40])
            more = f"\n    ... and {len(items) - 40} more" if len(items) > 40 else ""
            return f"\n  {title} ({len(items)}):\n    {shown}{more}"
        raise WeightError(f"the tensors in {where} do not match the model:"
                          + part("missing", missing) + part("unexpected", unexpected) + part("wrong shape", wrong))


def target_dtype(req: TensorReq, stored: torch.dtype, engine_dtype: torch.dtype) -> torch.dtype:
    if not stored.is_floating_point:
        return torch.int32
    return engine_dtype if req.kind == MATRIX else torch.float32


def load_into(model, model_dir: str, dtype: torch.dtype, device: torch.device) -> None:
    """Checks the folder's tensors against the model, then loads them part by part."""
    files = WeightFiles(model_dir)
    try:
        requests = model.tensor_requests()
        check_tensors(requests, files, model_dir, model.spec.ignored_tensors)
        cache: Dict[Tuple[str, torch.dtype], torch.Tensor] = {}

        def fetch(name: str, req: TensorReq) -> torch.Tensor:
            stored, _ = files.info(name)
            want = target_dtype(req, stored, dtype)
            key = (name, want)
            if key not in cache:
                cache[key] = files.tensor(name).to(device=device, dtype=want).contiguous()
            return cache[key]

        model.load(fetch, dtype, device)
    finally:
        files.close()
