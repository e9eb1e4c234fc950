"""One registry from an architecture's name to what builds it.

Name resolution follows crates/prelude-core/src/models/registry.rs:79-85,
:171-196 and crates/prelude-core/src/engine/config.rs:85-120: each entry of
``architectures`` is split at the first "For"; the prefix, stripped of
non-alphanumerics and lower-cased, is matched against the aliases; the suffix
must name causal-LM generation (the only task here).  ``model_type`` is the
fallback.
"""
from __future__ import annotations

import dataclasses
import re
from typing import Any, Callable, List, Mapping, Optional, Sequence


class UnknownArchitecture(ValueError):
    pass


@dataclasses.dataclass
class Architecture:
    name: str
    architecture_aliases: Sequence[str]
    model_type_aliases: Sequence[str]
    parse_config: Callable[[Mapping[str, Any]], Any]      # raw config.json -> typed configuration
    build_spec: Callable[[Any], Any]                       # typed configuration -> ModelSpec


_ARCHS: List[Architecture] = []


def _norm(s: str) -> str:
    return re.sub(r"[^0-9a-z]", "", s.lower())


def register_architecture(arch: Architecture) -> Architecture:
    for i, a in enumerate(_ARCHS):
        if a.name == arch.name:
            _ARCHS[i] = arch
            return arch
    _ARCHS.append(arch)
    return arch


def registered_architectures() -> List[str]:
    return [a.name for a in _ARCHS]


def _by_architecture_name(name: str) -> Optional[Architecture]:
    if "For" not in name:
        return None
    prefix, suffix = name.split("For", 1)
    if _norm(suffix) != "causallm":
        return None
    p = _norm(prefix)
    for a in _ARCHS:
        if p in (_norm(x) for x in a.architecture_aliases):
            return a
    return None


def resolve_architecture(raw: Mapping[str, Any]) -> Architecture:
    """The architecture a config.json names, or an error that says what was looked at."""
    names = raw.get("architectures") or []
    if isinstance(names, str):
        names = [names]
    for n in names:
        if isinstance(n, str):
            a = _by_architecture_name(n)
            if a is not None:
                return a
    mt = raw.get("model_type")
    if isinstance(mt, str):
        for a in _ARCHS:
            if _norm(mt) in (_norm(x) for x in a.model_type_aliases):
                return a
    raise UnknownArchitecture(
        f"unable to resolve model architecture from config metadata: architectures={list(names)!r}, "
        f"model_type={mt!r} (registered: {registered_architectures()})")
