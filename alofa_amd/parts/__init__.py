"""Parts a layer is put together from. Importing the package registers the
built-in kinds; ``register_part`` adds others (from anywhere, also from tests)."""
from .base import (SLOT, Block, CacheNeed, CacheTensor, FeedForward, Mixer, Norm, Part, PositionEncoding, Runtime, StateNeed,
                   build_part, part_class, register_part, tensors_of)
from . import attention, block, embedding, feed_forward, norm, position  # noqa: F401  (registration)

__all__ = ["SLOT", "Block", "CacheNeed", "CacheTensor", "FeedForward", "Mixer", "Norm", "Part", "PositionEncoding", "Runtime", "StateNeed",
           "build_part", "part_class", "register_part", "tensors_of"]
