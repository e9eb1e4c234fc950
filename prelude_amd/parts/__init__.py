"""The parts a layer is put together from.  Importing the package registers the built-in kinds."""
from .base import (MATRIX, NORM, VECTOR, Block, FeedForward, KVCacheSpec, Mixer, Norm, Part, PartError,
                   PositionEncoding, StateSpec, TensorReq, build_part, register_part, registered)
from . import attention, block, linear, mlp, norm, rope  # noqa: F401  (registration)

__all__ = ["MATRIX", "NORM", "VECTOR", "Block", "FeedForward", "KVCacheSpec", "Mixer", "Norm", "Part", "PartError",
           "PositionEncoding", "StateSpec", "TensorReq", "build_part", "register_part", "registered"]
