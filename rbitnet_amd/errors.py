"""Typed errors of the library, one per layer that can fail.

They play the part of the reference's `BitNetError` variants
(crates/bitnet-core/src/error.rs:6-27): every failure is a named error with a
message, never a crash of the process.
"""


class RbitnetError(Exception):
    """Base of every error this package raises on purpose."""


class ConfigError(RbitnetError):
    """config.json is missing a key, holds an invalid value, or names an
    architecture or option that is not supported."""


class WeightError(RbitnetError):
    """The weight file is malformed, or its tensors do not match the model:
    the message lists missing and unexpected tensors and wrong shapes."""


class CacheError(RbitnetError):
    """A slot or page was asked for that is not there, or given back twice."""


class InferenceError(RbitnetError):
    """A step was asked for that cannot run: token id out of range, position
    beyond the model's or the cache's limit, malformed batch."""


class KernelError(RbitnetError):
    """The HIP extension is missing or refuses a size it cannot compute."""
