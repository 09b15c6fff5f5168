"""How the parts of one layer are arranged.

"prenorm" (crates/bitnet-core/src/llama/model.rs:236-307):
    x += mixer(norm1(x));  x += feed_forward(norm2(x))
The residual stream x is float32 and each sum is done by the norm that follows it (see
norm.py), so a block takes the previous block's not yet added output as `pending` and
returns its own.  The model adds the last one in the final norm.

Who adds what to the stream, and in which form a part's output travels to the next norm, is
`stream.py`'s business: an arrangement calls `sublayer(part, norm, x, pending, next_norm, ...)`
once per part and hands on what comes back.

Interface of a block: parts() -> {name: part} for the loader (names are tensor-name
segments below the layer's prefix); mixer (for the cache request);
forward(x, pending, ctx, view) -> pending (a tensor still to be added, None, or GainedRows).
A block may offer first_norm (the norm its forward begins with) and say takes_next_norm:
forward then also takes next_norm, the first norm of whatever runs after it.
"""
from __future__ import annotations

from typing import Dict

import torch

from .base import BuildEnv, build_part, register_block
from .stream import normed_for, sublayer  # noqa: F401  (normed_for: its old home)

DEFAULT_SEGMENTS = {"norm1": "input_layernorm", "mixer": "self_attn", "norm2": "post_attention_layernorm",
                    "feed_forward": "mlp"}


class PreNormBlock:
    takes_next_norm = True

    def __init__(self, layer_spec, env: BuildEnv):
        self.norm1 = build_part("norm", layer_spec.norm1, env)
        self.mixer = build_part("mixer", layer_spec.mixer, env)
        self.norm2 = build_part("norm", layer_spec.norm2, env)
        self.feed_forward = build_part("feed_forward", layer_spec.feed_forward, env)
        self.segments = dict(DEFAULT_SEGMENTS, **(getattr(layer_spec, "segments", None) or {}))

    @property
    def graph_safe(self) -> bool:
        return all(getattr(p, "graph_safe", False) for p in (self.norm1, self.mixer, self.norm2, self.feed_forward))

    @property
    def plan_safe(self) -> bool:
        return all(getattr(p, "plan_safe", False) for p in (self.norm1, self.mixer, self.norm2, self.feed_forward))

    def parts(self) -> Dict[str, object]:
        return {self.segments["norm1"]: self.norm1, self.segments["mixer"]: self.mixer,
                self.segments["norm2"]: self.norm2, self.segments["feed_forward"]: self.feed_forward}

    @property
    def first_norm(self):
        return self.norm1

    def forward(self, x: torch.Tensor, pending, ctx, view, next_norm=None):
        a = sublayer(self.mixer, self.norm1, x, pending, self.norm2, ctx, view)
        return sublayer(self.feed_forward, self.norm2, x, a, next_norm, ctx)


register_block("prenorm", PreNormBlock)
