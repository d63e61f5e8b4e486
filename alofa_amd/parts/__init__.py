"""Parts a layer is put together from. Importing the package registers the
built-in kinds; ``register_part`` adds others (from anywhere, also from tests)."""
from .base import (SLOT, Block, CacheNeed, CacheTensor, FeedForward, Join, Mixer, Norm, Part, PositionEncoding, Runtime, StateNeed, TimeConv,
                   build_part, part_class, register_part, tensors_of)
from . import attention, block, conv, embedding, feed_forward, join, latent, mixture, norm, position, recurrent, talking, window  # noqa: F401  (registration)

__all__ = ["SLOT", "Block", "CacheNeed", "CacheTensor", "FeedForward", "Join", "Mixer", "Norm", "Part", "PositionEncoding", "Runtime", "StateNeed", "TimeConv",
           "build_part", "part_class", "register_part", "tensors_of"]
