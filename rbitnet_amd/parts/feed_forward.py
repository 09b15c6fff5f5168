"""The SiLU-gated feed-forward.

Reference (crates/bitnet-core/src/llama/model.rs:296-306): g = silu(Wgate h) with
silu(v) = v / (1 + exp(-v)) (:116-120), u = Wup h, out = Wdown (g * u).  No biases.
Gate and up share one product; on the matrix cores the gate is applied in that
product's epilogue, on the generic path by a small kernel on its float32 result.

Parameters: intermediate_size, activation ("silu"), names.
Interface of a feed-forward: tensor_specs() / load(tensors) / forward(h [T, E], ctx) ->
float32 [T, E].  It may say `takes_gained_rows` and `adds_to_stream` of itself as a mixer
may (this one does both).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..errors import ConfigError
from .base import BuildEnv, Part, TensorSpec, register_feed_forward
from .linear import can_fuse_gate, gated_linear, linear_to_stream, pack_gate_up, pack_rows

DEFAULT_NAMES = {"gate": "gate_proj.weight", "up": "up_proj.weight", "down": "down_proj.weight"}


class SwiGLU(Part):
    graph_safe = True
    plan_safe = True
    takes_gained_rows = True
    adds_to_stream = True

    def __init__(self, params: Dict, env: BuildEnv):
        self.env = env
        self.ff = int(params["intermediate_size"])
        if params.get("activation", "silu") != "silu":
            raise ConfigError(f"feed-forward activation {params.get('activation')!r} not supported (silu)")
        self.names = dict(DEFAULT_NAMES, **(params.get("names") or {}))
        self.hidden = env.hidden_size
        self.fused = can_fuse_gate(env.dtype, self.hidden, self.ff) and not getattr(env, "generic_only", False)
        self.w_gate_up: Optional[torch.Tensor] = None
        self.w_down: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {self.names["gate"]: TensorSpec((self.ff, self.hidden)),
                self.names["up"]: TensorSpec((self.ff, self.hidden)),
                self.names["down"]: TensorSpec((self.hidden, self.ff))}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        allowed = not getattr(self.env, "generic_only", False)
        self.w_gate_up = pack_gate_up(self.env.lib, tensors[self.names["gate"]], tensors[self.names["up"]], self.fused,
                                      allowed)
        down = tensors[self.names["down"]]
        self.w_down = pack_rows(self.env.lib, [(down, 0, None, None)], down.shape[0], down.shape[1], down.dtype,
                                down.device, allowed)

    def forward(self, h, ctx=None, stream: Optional[torch.Tensor] = None, next_norm=None):
        lib = self.env.lib
        t = gated_linear(lib, h, self.w_gate_up, self.ff, self.fused)
        return linear_to_stream(lib, t, self.w_down, stream, next_norm)


register_feed_forward("swiglu", SwiGLU)
