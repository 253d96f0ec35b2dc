"""The parts a layer is put together from.  Importing the package registers the built-in kinds."""
from .base import (MATRIX, NORM, TABLE, VECTOR, Block, FeedForward, KVCacheSpec, KVLayerCache, LatentCacheSpec, LatentLayerCache, Mixer, Norm, PagedCacheSpec, Part,
                   PartError, PositionEncoding, SlotCacheSpec, StateLayerCache, StateSpec, TensorReq, build_part,
                   register_part, registered)
from . import attention, block, conv_input, delta_rule, experts, latent_attention, lightning, linear, mlp, norm, parallel, rope  # noqa: F401  (registration)

__all__ = ["MATRIX", "NORM", "TABLE", "VECTOR", "Block", "FeedForward", "KVCacheSpec", "KVLayerCache", "LatentCacheSpec", "LatentLayerCache", "Mixer", "Norm",
           "PagedCacheSpec", "Part", "PartError", "PositionEncoding", "SlotCacheSpec", "StateLayerCache", "StateSpec",
           "TensorReq", "build_part", "register_part", "registered"]
