from .base import (BuildEnv, CacheRequest, Part, TensorSpec, build_part, register_block, register_feed_forward,
                   register_mixer, register_norm, register_position, registered)
from . import norm, position, attention, feed_forward, block  # noqa: F401  (registers the built-in kinds)

__all__ = ["BuildEnv", "CacheRequest", "Part", "TensorSpec", "build_part", "register_block",
           "register_feed_forward", "register_mixer", "register_norm", "register_position", "registered"]
