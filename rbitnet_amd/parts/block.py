"""How the parts of one layer are arranged.

"prenorm" (crates/bitnet-core/src/llama/model.rs:236-307):
    x += mixer(norm1(x));  x += feed_forward(norm2(x))
The residual stream x is float32 and each sum is done by the norm that follows it (see
norm.py), so a block takes the previous block's not yet added output as `pending` and
returns its own.  The model adds the last one in the final norm.

A part that says `adds_to_stream` is given the stream and the norm that follows and may add
its output itself; it then returns None, or the rows as its last product prepared them for
that norm (`GainedRows`), which go to the next part if it says `takes_gained_rows`.  With
both, a step of a few tokens runs no kernel between the products.

Interface of a block: parts() -> {name: part} for the loader (names are tensor-name
segments below the layer's prefix); mixer (for the cache request);
forward(x, pending, ctx, view) -> pending (a tensor still to be added, None, or GainedRows).
A block may offer first_norm (the norm its forward begins with) and say takes_next_norm:
forward then also takes next_norm, the first norm of whatever runs after it.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import BuildEnv, build_part, register_block
from .norm import GainedRows

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

    def parts(self) -> Dict[str, object]:
        return {self.segments["norm1"]: self.norm1, self.segments["mixer"]: self.mixer,
                self.segments["norm2"]: self.norm2, self.segments["feed_forward"]: self.feed_forward}

    @property
    def first_norm(self):
        return self.norm1

    def forward(self, x: torch.Tensor, pending, ctx, view, next_norm=None):
        h = normed_for(self.mixer, self.norm1, x, pending)
        if getattr(self.mixer, "adds_to_stream", False):
            a = self.mixer.forward(h, ctx, view, stream=x, next_norm=self.norm2)
        else:
            a = self.mixer.forward(h, ctx, view)
        h2 = normed_for(self.feed_forward, self.norm2, x, a)
        if getattr(self.feed_forward, "adds_to_stream", False):
            return self.feed_forward.forward(h2, ctx, stream=x, next_norm=next_norm)
        return self.feed_forward.forward(h2, ctx)


def normed_for(part, norm, x: torch.Tensor, pending, rows: Optional[torch.Tensor] = None):
    """The input of `part`: the stream x, with `pending` added if that is a tensor, normalised
    by `norm` (all rows, or `rows`).  GainedRows that were made for this norm go on as they are
    to a part that takes them."""
    if isinstance(pending, GainedRows):
        if pending.norm is norm and getattr(part, "takes_gained_rows", False):
            return pending.select(rows)
        return norm.forward(x, None, rows)         # the stream holds the sum already
    return norm.forward(x, pending, rows)


register_block("prenorm", PreNormBlock)
