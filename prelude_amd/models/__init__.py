"""Model specifications and the generic decoder built from them.  Importing registers the architectures."""
from .spec import LayerSpec, ModelSpec, PartSpec, RunSpec
from . import qwen3  # noqa: F401  (registration)

__all__ = ["LayerSpec", "ModelSpec", "PartSpec", "RunSpec"]
