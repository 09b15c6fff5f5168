"""What every part is: a kind name, parameters, tensors it owns, a forward.

Kinds of parts and the registry each lives in:

* norm            `register_norm`           forward(x_f32 [T, E], delta, rows) -> h [rows, E]
* position        `register_position`       a table or rule keyed by absolute position
* mixer           `register_mixer`          forward(h [T, E], ctx, view) -> [T, E_out]
* feed-forward    `register_feed_forward`   forward(h [T, E], ctx) -> [T, E]
* block           `register_block`          arranges norm, mixer, norm, feed-forward
* embedding       `register_embedding`      forward(ctx) -> x [T, E], the residual stream
* head            `register_head`           forward(x, pending, rows, ctx) -> logits [rows, V]

A part is built from `(params, env)`: `params` is the dict of its `PartSpec`,
`env` a `BuildEnv` (model width, compute dtype, device, the kernel library).
It declares its tensors (`tensor_specs`) with names relative to its own prefix,
and receives them in `load`.  A mixer further declares what it needs of the
cache (`cache_request`).  No part sees the configuration it came from or the
model it is in.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Dict, Optional, Tuple

import torch

from ..errors import ConfigError


@dataclass(frozen=True)
class TensorSpec:
    """A tensor a part owns.

    role "matrix": held in the compute dtype (bfloat16 or float32);
    role "gain":   a norm's gain, held in float32 (widening is exact);
    role "table":  integers, held as int32.
    init names the random initialisation: "normal" is N(0, std), "ones_normal"
    is 1 + N(0, norm_std)."""
    shape: Tuple[int, ...]
    role: str = "matrix"
    init: str = "normal"


@dataclass
class BuildEnv:
    hidden_size: int
    dtype: torch.dtype
    device: torch.device
    lib: Any                    # rbitnet_amd.csrc.lib.Kernels (None when only shapes are wanted)
    layer_index: int = -1
    # one dictionary for all layers of a model: read-only data (tables) that parts with equal
    # parameters build once and share, keyed by the part
    shared: Dict[Any, Any] = field(default_factory=dict)
    generic_only: bool = False            # never the matrix-core kernels (tests of the generic ones)
    max_seq_len: Optional[int] = None     # the longest sequence the engine will run, if it is known


@dataclass
class CacheRequest:
    """What a mixer needs of the cache.

    kind "kv":    keys and values per token, `heads` x `head_dim` each; `window`
                  (None = all) is how far back a query looks, so that pages
                  behind it can be given back.
    kind "state": `state_shape` numbers per sequence, set to `state_init` when a
                  slot is handed out.
    Layers with equal requests share one group of storage."""
    kind: str
    heads: int = 0
    head_dim: int = 0
    window: Optional[int] = None
    state_shape: Tuple[int, ...] = ()
    state_init: float = 0.0
    state_dtype: torch.dtype = torch.float32

    def key(self) -> Tuple:
        return (self.kind, self.heads, self.head_dim, self.window, tuple(self.state_shape),
                self.state_init, self.state_dtype)


class Part:
    # True when forward only launches kernels on the current stream (no host
    # synchronisation, no host-side reads of device data): the decode step may then be
    # captured into a HIP graph.  A part that does not say so is run launch by launch.
    graph_safe = False
    # True when forward does nothing on the device but call the kernel library (no torch operation of
    # its own that computes or copies): the launches of a step can then be recorded in the library and
    # issued again from C++ for the next step of the same shape.
    plan_safe = False

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        pass


_REGISTRIES: Dict[str, Dict[str, Callable[..., Any]]] = {
    "norm": {}, "position": {}, "mixer": {}, "feed_forward": {}, "block": {}, "embedding": {}, "head": {},
}


def _register(group: str, kind: str, factory: Callable[..., Any]) -> None:
    _REGISTRIES[group][kind] = factory


def register_norm(kind: str, factory: Callable[..., Any]) -> None:
    _register("norm", kind, factory)


def register_position(kind: str, factory: Callable[..., Any]) -> None:
    _register("position", kind, factory)


def register_mixer(kind: str, factory: Callable[..., Any]) -> None:
    _register("mixer", kind, factory)


def register_feed_forward(kind: str, factory: Callable[..., Any]) -> None:
    _register("feed_forward", kind, factory)


def register_block(kind: str, factory: Callable[..., Any]) -> None:
    _register("block", kind, factory)


def register_embedding(kind: str, factory: Callable[..., Any]) -> None:
    _register("embedding", kind, factory)


def register_head(kind: str, factory: Callable[..., Any]) -> None:
    _register("head", kind, factory)


def build_part(group: str, spec: Any, env: BuildEnv) -> Any:
    table = _REGISTRIES[group]
    if spec.kind not in table:
        raise ConfigError(f"unknown {group} kind {spec.kind!r}; registered: {', '.join(sorted(table))}")
    return table[spec.kind](spec.params, env)


def registered(group: str):
    return sorted(_REGISTRIES[group])
