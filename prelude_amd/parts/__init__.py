"""The parts a layer is put together from.  Importing the package registers the built-in kinds."""
from .base import (MATRIX, NORM, VECTOR, Block, FeedForward, KVCacheSpec, KVLayerCache, Mixer, Norm, PagedCacheSpec, Part,
                   PartError, PositionEncoding, SlotCacheSpec, StateLayerCache, StateSpec, TensorReq, build_part,
                   register_part, registered)
from . import attention, block, linear, mlp, norm, rope  # noqa: F401  (registration)

__all__ = ["MATRIX", "NORM", "VECTOR", "Block", "FeedForward", "KVCacheSpec", "KVLayerCache", "Mixer", "Norm",
           "PagedCacheSpec", "Part", "PartError", "PositionEncoding", "SlotCacheSpec", "StateLayerCache", "StateSpec",
           "TensorReq", "build_part", "register_part", "registered"]
