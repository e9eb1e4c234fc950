"""Reading and writing safetensors files by tensor name, without loading what is not asked for.

File layout: 8 bytes little-endian header length N, N bytes of JSON
``{name: {"dtype", "shape", "data_offsets": [begin, end]}, "__metadata__": {...}}``,
then the tensors' bytes.  Which files make up a model follows
crates/prelude-core/src/engine/weights.rs:57-144: ``model.safetensors.index.json``
(its ``weight_map`` values, absolute paths and ``..`` refused), else
``model.safetensors``, else every ``*.safetensors`` in name order.
"""
from __future__ import annotations

import json
import mmap
import os
import struct
from typing import Dict, List, Tuple

import torch

_DTYPES = {
    "F64": torch.float64, "F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16,
    "I64": torch.int64, "I32": torch.int32, "I16": torch.int16, "I8": torch.int8, "U8": torch.uint8,
    "BOOL": torch.bool,
}
_NAMES = {v: k for k, v in _DTYPES.items()}


class WeightFileError(ValueError):
    pass


class SafetensorsFile:
    """One file, memory-mapped; tensors are materialised one at a time."""

    def __init__(self, path: str):
        self.path = path
        try:
            self._fh = open(path, "rb")
        except OSError as e:
            raise WeightFileError(f"cannot open {path}: {e}") from None
        size = os.fstat(self._fh.fileno()).st_size
        if size < 8:
            raise WeightFileError(f"{path}: too short to be a safetensors file")
        (n,) = struct.unpack("<Q", self._fh.read(8))
        if n > size - 8:
            raise WeightFileError(f"{path}: header length {n} exceeds the file")
        try:
            header = json.loads(self._fh.read(n).decode("utf-8"))
        except (UnicodeDecodeError, json.JSONDecodeError) as e:
            raise WeightFileError(f"{path}: header is not JSON: {e}") from None
        self.metadata = header.pop("__metadata__", {}) or {}
        self._base = 8 + n
        self.entries: Dict[str, Tuple[torch.dtype, Tuple[int, ...], int, int]] = {}
        for name, e in header.items():
            try:
                dt = _DTYPES[e["dtype"]]
                shape = tuple(int(s) for s in e["shape"])
                b, en = (int(x) for x in e["data_offsets"])
            except (KeyError, TypeError, ValueError):
                raise WeightFileError(f"{path}: bad header entry for tensor {name!r}") from None
            count = 1
            for s in shape:
                count *= s
            if en - b != count * torch.empty((), dtype=dt).element_size() or b < 0 or self._base + en > size:
                raise WeightFileError(f"{path}: tensor {name!r} has offsets [{b}, {en}) that do not fit its shape "
                                      f"{shape} or the file")
            self.entries[name] = (dt, shape, b, en)
        # a private copy-on-write mapping: writable for torch, the file itself is never touched
        self._mm = mmap.mmap(self._fh.fileno(), 0, access=mmap.ACCESS_COPY) if size > 0 else None

    def names(self) -> List[str]:
        return list(self.entries)

    def info(self, name: str) -> Tuple[torch.dtype, Tuple[int, ...]]:
        dt, shape, _, _ = self.entries[name]
        return dt, shape

    def tensor(self, name: str) -> torch.Tensor:
        """A CPU tensor viewing the mapped bytes (copy it before the file is closed)."""
        dt, shape, b, e = self.entries[name]
        if e == b:
            return torch.empty(shape, dtype=dt)
        flat = torch.frombuffer(self._mm, dtype=torch.uint8, count=e - b, offset=self._base + b)
        return flat.view(dt).reshape(shape)

    def close(self) -> None:
        # tensors handed out may still view the mapping; let the garbage collector end it
        self._mm = None
        self._fh.close()


def find_safetensor_files(model_dir: str) -> List[str]:
    index = os.path.join(model_dir, "model.safetensors.index.json")
    if os.path.isfile(index):
        try:
            with open(index, "r", encoding="utf-8") as f:
                weight_map = json.load(f)["weight_map"]
        except (OSError, KeyError, json.JSONDecodeError, TypeError) as e:
            raise WeightFileError(f"{index}: cannot read weight_map: {e}") from None
        files: List[str] = []
        for fn in weight_map.values():
            if not isinstance(fn, str) or os.path.isabs(fn) or ".." in fn.replace("\\", "/").split("/"):
                raise WeightFileError(f"{index}: refusing shard path {fn!r}")
            if fn not in files:
                files.append(fn)
        return [os.path.join(model_dir, f) for f in files]
    single = os.path.join(model_dir, "model.safetensors")
    if os.path.isfile(single):
        return [single]
    try:
        found = sorted(f for f in os.listdir(model_dir) if f.endswith(".safetensors"))
    except OSError as e:
        raise WeightFileError(f"cannot list model folder {model_dir!r}: {e}") from None
    if not found:
        raise WeightFileError(f"no .safetensors files were resolved in {model_dir!r}")
    return [os.path.join(model_dir, f) for f in found]


class WeightFiles:
    """All tensors of a model folder by name."""

    def __init__(self, model_dir: str):
        self.files = [SafetensorsFile(p) for p in find_safetensor_files(model_dir)]
        self._where: Dict[str, SafetensorsFile] = {}
        for f in self.files:
            for n in f.names():
                if n in self._where:
                    raise WeightFileError(f"tensor {n!r} appears in both {self._where[n].path} and {f.path}")
                self._where[n] = f

    def names(self) -> List[str]:
        return list(self._where)

    def __contains__(self, name: str) -> bool:
        return name in self._where

    def info(self, name: str):
        return self._where[name].info(name)

    def tensor(self, name: str) -> torch.Tensor:
        return self._where[name].tensor(name)

    def close(self) -> None:
        for f in self.files:
            f.close()


def write_safetensors(path: str, tensors: Dict[str, torch.Tensor], metadata: Dict[str, str] | None = None) -> None:
    """Writes CPU tensors in name order; the data section starts 8-byte aligned."""
    header: Dict[str, dict] = {}
    if metadata:
        header["__metadata__"] = {str(k): str(v) for k, v in metadata.items()}
    offset = 0
    order = sorted(tensors)
    for name in order:
        t = tensors[name]
        if t.dtype not in _NAMES:
            raise WeightFileError(f"tensor {name!r}: element type {t.dtype} cannot be stored")
        nbytes = t.numel() * t.element_size()
        header[name] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [offset, offset + nbytes]}
        offset += nbytes
    blob = json.dumps(header, separators=(",", ":")).encode("utf-8")
    blob += b" " * ((8 - len(blob) % 8) % 8)
    tmp = path + f".tmp{os.getpid()}"
    with open(tmp, "wb") as f:
        f.write(struct.pack("<Q", len(blob)))
        f.write(blob)
        for name in order:
            t = tensors[name].detach().cpu().contiguous()
            f.write(t.reshape(-1).view(torch.uint8).numpy().tobytes() if t.numel() else b"")
    os.replace(tmp, path)
