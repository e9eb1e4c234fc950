"""Shared by the GPU tests: tiny model folders in temporary places, the plain implementation's logits, schedules."""
import functools
import json
import os
import tempfile

import torch

import plain_model as pm

CONFIGS = {"a": pm.tiny_config_a, "b": pm.tiny_config_b, "c": pm.tiny_config_c}
# (seed, matrix std, norm-scale std) of each configuration's weights
WEIGHT_STATS = {"a": (0, 0.02, 0.01), "b": (1, 0.05, 0.05), "c": (2, 0.05, 0.03)}
PAGE = {"a": 8, "b": 16, "c": 8}
_keep = []


@functools.lru_cache(maxsize=None)
def model_folder(name: str, stored: str = "float32"):
    """(folder, config dict, weights dict in float32) of a tiny model written by the test suite's own generator."""
    from prelude_amd.weights import write_safetensors
    cfg = CONFIGS[name]()
    seed, std, nstd = WEIGHT_STATS[name]
    w = pm.random_weights(cfg, seed=seed, std=std, norm_std=nstd)
    tmp = tempfile.TemporaryDirectory(prefix=f"prelude_amd_test_{name}_")
    _keep.append(tmp)
    with open(os.path.join(tmp.name, "config.json"), "w") as f:
        json.dump(cfg, f)
    dt = torch.float32 if stored == "float32" else torch.bfloat16
    write_safetensors(os.path.join(tmp.name, "model.safetensors"), {k: v.to(dt) for k, v in w.items()})
    if stored != "float32":
        w = {k: v.to(dt).float() for k, v in w.items()}
    return tmp.name, cfg, w


@functools.lru_cache(maxsize=None)
def reference_logits(name: str, seed: int, length: int, stored: str = "float32"):
    """(tokens, float64 logits [length, vocab]) of the plain implementation for a seeded random sequence."""
    _, cfg, w = model_folder(name, stored)
    g = torch.Generator().manual_seed(1000 + seed)
    toks = torch.randint(0, cfg["vocab_size"], (length,), generator=g).tolist()
    return toks, pm.forward(cfg, w, toks)


def tolerance(dtype: str, ref: torch.Tensor) -> float:
    """Largest allowed |engine - plain| over a tensor of logits.  float32: rounding of a few hundred 32-bit
    operations per logit.  bfloat16: a tenth of the logits' spread (their standard deviation).  Every activation
    is rounded to 8 bits of mantissa, which adds up to a few hundredths of the spread by the last layer: over the
    three tiny configurations and sixty drawn ones the largest error measured was 0.03 to 0.063 of it.  A key
    that is lost, misplaced or taken from another request moves a logit by a quarter of the spread or more, in
    every configuration; a bound tied to the largest logit instead would let that pass where logits are small."""
    if dtype == "float32":
        return 1e-5 * max(1.0, float(ref.abs().max()))
    return 0.1 * float(ref.double().std())


def check(got, ref, dtype, what=""):
    got = torch.as_tensor(got).double().reshape(ref.shape)
    err = (got - ref).abs()
    worst = int(err.reshape(len(ref), -1).max(dim=1).values.argmax()) if ref.dim() > 1 else 0
    assert float(err.max()) <= tolerance(dtype, ref), \
        f"{what}: max |engine - plain| = {float(err.max()):.3e} > {tolerance(dtype, ref):.3e}; first bad row {worst}"
