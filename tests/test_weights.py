"""Safetensors reading and writing, the loader's one error, the random-weights mode (no GPU)."""
import json
import os
import struct

import pytest
import torch

import plain_model as pm
from prelude_amd import models  # noqa: F401
from prelude_amd.config import resolve_architecture
from prelude_amd.models.causal_lm import CausalLM
from prelude_amd.weights import (WeightError, WeightFileError, WeightFiles, check_tensors, find_safetensor_files,
                                 random_tensors, write_random_model, write_safetensors)
from prelude_amd.weights.loader import target_dtype
from prelude_amd.parts.base import MATRIX, NORM, TensorReq


def _model(raw):
    arch = resolve_architecture(raw)
    return CausalLM(arch.build_spec(arch.parse_config(raw)))


def test_roundtrip_and_interop(tmp_path):
    t = {"a": torch.randn(3, 5).to(torch.bfloat16), "b.c": torch.arange(7, dtype=torch.int32),
         "d": torch.randn(2, 2, 2), "e": torch.zeros(0, 4)}
    path = str(tmp_path / "model.safetensors")
    write_safetensors(path, t, {"k": "v"})
    f = WeightFiles(str(tmp_path))
    assert sorted(f.names()) == sorted(t)
    for n, x in t.items():
        assert f.info(n) == (x.dtype, tuple(x.shape))
        assert torch.equal(f.tensor(n), x)
    # the same bytes read by the safetensors package, and its files read by us
    from safetensors.torch import load_file, save_file
    theirs = load_file(path)
    assert all(torch.equal(theirs[n], t[n]) for n in t)
    save_file({n: x.contiguous() for n, x in t.items()}, str(tmp_path / "other.safetensors"))
    from prelude_amd.weights import SafetensorsFile
    g = SafetensorsFile(str(tmp_path / "other.safetensors"))
    assert all(torch.equal(g.tensor(n), t[n]) for n in t)


def test_file_discovery(tmp_path):
    # crates/prelude-core/src/engine/weights.rs:57-144
    with pytest.raises(WeightFileError, match="no .safetensors"):
        find_safetensor_files(str(tmp_path))
    write_safetensors(str(tmp_path / "b.safetensors"), {"x": torch.zeros(1)})
    write_safetensors(str(tmp_path / "a.safetensors"), {"y": torch.zeros(1)})
    assert [os.path.basename(p) for p in find_safetensor_files(str(tmp_path))] == ["a.safetensors", "b.safetensors"]
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {"x": "b.safetensors", "y": "a.safetensors", "z": "b.safetensors"}}))
    assert [os.path.basename(p) for p in find_safetensor_files(str(tmp_path))] == ["b.safetensors", "a.safetensors"]
    for bad in ("/etc/passwd", "../x.safetensors", "sub/../../x.safetensors"):
        (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"weight_map": {"x": bad}}))
        with pytest.raises(WeightFileError, match="refusing"):
            find_safetensor_files(str(tmp_path))


def test_corrupt_files(tmp_path):
    p = tmp_path / "model.safetensors"
    p.write_bytes(b"abc")
    with pytest.raises(WeightFileError, match="too short"):
        WeightFiles(str(tmp_path))
    p.write_bytes(struct.pack("<Q", 1000) + b"{}")
    with pytest.raises(WeightFileError, match="exceeds"):
        WeightFiles(str(tmp_path))
    hdr = json.dumps({"x": {"dtype": "F32", "shape": [4], "data_offsets": [0, 8]}}).encode()
    p.write_bytes(struct.pack("<Q", len(hdr)) + hdr + b"\0" * 8)
    with pytest.raises(WeightFileError, match="do not fit"):
        WeightFiles(str(tmp_path))


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    raw = pm.tiny_config_b()
    t = random_tensors(raw, seed=0, dtype=torch.float32)
    del t["model.layers.1.mlp.up_proj.weight"]
    del t["lm_head.weight"]
    t["model.layers.0.self_attn.q_norm.weight"] = torch.zeros(16)
    t["model.layers.2.self_attn.k_proj.weight"] = torch.zeros(32, 95)
    t["model.layers.7.extra.weight"] = torch.zeros(2)
    write_safetensors(str(tmp_path / "model.safetensors"), t)
    files = WeightFiles(str(tmp_path))
    with pytest.raises(WeightError) as ei:
        check_tensors(_model(raw).tensor_requests(), files, "X")
    msg = str(ei.value)
    assert "missing (2)" in msg and "model.layers.1.mlp.up_proj.weight" in msg and "lm_head.weight" in msg
    assert "unexpected (1)" in msg and "model.layers.7.extra.weight" in msg
    assert "wrong shape (2)" in msg and "expected [32], got [16]" in msg and "expected [32, 96], got [32, 95]" in msg


def test_tensors_an_architecture_knows_of_and_does_not_read_are_passed_over(tmp_path):
    """A tied checkpoint that still carries its unused head, and exported rotary frequencies, load (the reference
    fetches by name and never looks at them: crates/prelude-core/src/models/qwen3.rs:637-643,
    crates/prelude-core/src/engine/weight_loader.rs:200-285); anything else nothing asks for is still reported."""
    raw = pm.tiny_config_a()
    t = random_tensors(raw, seed=0)
    assert "lm_head.weight" not in t
    t["lm_head.weight"] = torch.zeros(256, 64)
    t["model.layers.1.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    write_safetensors(str(tmp_path / "model.safetensors"), t)
    model = _model(raw)
    assert model.spec.ignored_tensors == ("*.rotary_emb.inv_freq", "lm_head.weight")
    check_tensors(model.tensor_requests(), WeightFiles(str(tmp_path)), "X", model.spec.ignored_tensors)
    with pytest.raises(WeightError, match=r"unexpected \(2\)"):      # without the architecture's say-so: reported
        check_tensors(model.tensor_requests(), WeightFiles(str(tmp_path)), "X")
    t["model.layers.0.mlp.gate_up_proj.weight"] = torch.zeros(4)
    write_safetensors(str(tmp_path / "model.safetensors"), t)
    with pytest.raises(WeightError, match=r"unexpected \(1\)") as ei:
        check_tensors(model.tensor_requests(), WeightFiles(str(tmp_path)), "X", model.spec.ignored_tensors)
    assert "gate_up_proj" in str(ei.value) and "lm_head" not in str(ei.value)
    # an untied model asks for its head: nothing is passed over there but the frequencies
    assert _model(pm.tiny_config_b()).spec.ignored_tensors == ("*.rotary_emb.inv_freq",)


def test_device_types():
    bf, f32 = torch.bfloat16, torch.float32
    assert target_dtype(TensorReq((2, 2), MATRIX), bf, bf) == bf
    assert target_dtype(TensorReq((2, 2), MATRIX), f32, bf) == bf
    assert target_dtype(TensorReq((2, 2), MATRIX), bf, f32) == f32
    assert target_dtype(TensorReq((2,), NORM), bf, bf) == f32       # small vectors are always 32-bit
    assert target_dtype(TensorReq((2,), NORM), f32, bf) == f32      # stored in 32-bit stays so
    assert target_dtype(TensorReq((2,), MATRIX), torch.int64, bf) == torch.int32


def test_random_weights_mode(tmp_path):
    raw = pm.tiny_config_c()
    d = write_random_model(raw, str(tmp_path / "m"), seed=11, std=0.05, norm_std=0.02, dtype=torch.float32)
    assert json.load(open(os.path.join(d, "config.json")))["head_dim"] == 48
    f = WeightFiles(d)
    assert set(f.names()) == set(pm.tensor_shapes(raw))
    for n, s in pm.tensor_shapes(raw).items():
        assert f.info(n) == (torch.float32, tuple(s))
    w = f.tensor("model.layers.0.mlp.gate_proj.weight")
    assert abs(float(w.std()) - 0.05) < 0.005 and abs(float(w.mean())) < 0.005
    nw = f.tensor("model.norm.weight")
    assert abs(float(nw.mean()) - 1.0) < 0.02 and 0.005 < float(nw.std()) < 0.04
    # same seed, same tensors; other seed, other tensors; a tensor does not depend on the rest of the model
    again = random_tensors(raw, seed=11, std=0.05, norm_std=0.02, dtype=torch.float32)
    assert all(torch.equal(again[n], f.tensor(n)) for n in again)
    other = random_tensors(raw, seed=12, std=0.05, norm_std=0.02, dtype=torch.float32)
    assert not torch.equal(other["model.norm.weight"], again["model.norm.weight"])
    fewer = random_tensors(dict(raw, num_hidden_layers=2, max_window_layers=2), seed=11, std=0.05, norm_std=0.02, dtype=torch.float32)
    assert torch.equal(fewer["model.layers.1.mlp.up_proj.weight"], again["model.layers.1.mlp.up_proj.weight"])
    # the plain implementation runs on what was written
    lg = pm.forward(raw, {n: f.tensor(n) for n in f.names()}, [1, 2, 3, 4])
    assert lg.shape == (4, 331) and float(lg.abs().max()) > 0
    assert f.info("model.embed_tokens.weight")[0] == torch.float32
    d2 = write_random_model(raw, str(tmp_path / "m2"), seed=11)
    assert WeightFiles(d2).info("model.embed_tokens.weight")[0] == torch.bfloat16
