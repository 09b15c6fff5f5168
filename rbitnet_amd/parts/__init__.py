from .base import (BuildEnv, CacheRequest, Part, TensorSpec, build_part, register_block, register_embedding,
                   register_feed_forward, register_head, register_mixer, register_norm, register_position, registered)
from . import norm, position, attention, feed_forward, block, ends  # noqa: F401  (registers the built-in kinds)

__all__ = ["BuildEnv", "CacheRequest", "Part", "TensorSpec", "build_part", "register_block", "register_embedding",
           "register_feed_forward", "register_head", "register_mixer", "register_norm", "register_position",
           "registered"]
