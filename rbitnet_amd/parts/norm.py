"""RMS norm with the residual add folded in.

Reference: s = sum(x^2) / n; y_i = x_i * w_i / sqrt(s + eps), eps inside the root, the
gain multiplies directly (crates/bitnet-core/src/llama/model.rs:93-100).  The residual
sums of model.rs:292-294 and :304-306 are done by the norm that follows them: the
stream x is float32, `delta` (the previous part's output, float32) is added in place
and the normalised rows come back in the compute dtype.

Interface of a norm: forward(x, delta=None, rows=None) -> h
  x      float32 [T, E], the residual stream; updated in place when delta is given
  delta  float32 [T, E] or None; a norm that says `adds_terms` also takes [P, T, E], P terms
         to be added up in their order
  rows   int32 [R] or None: normalise only these rows (x is then left as it is)

A norm that says `folds_into_products` (with weight, eps and size as here) lets the product
before it and the product after it do its work when a step has few tokens: the first, which
adds to the stream, also leaves bf16(x * gain) and the sums of x^2 (`GainedRows`); the second
takes these as its tokens and multiplies its result by 1 / sqrt(mean(x^2) + eps).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .base import BuildEnv, Part, TensorSpec, register_norm
from .stream import GainedRows  # noqa: F401  (its old home; importers find it here too)


class RMSNorm(Part):
    graph_safe = True
    plan_safe = True
    folds_into_products = True
    adds_terms = True

    def __init__(self, params: Dict, env: BuildEnv):
        self.size = int(params["size"])
        self.eps = float(params["eps"])
        self.env = env
        self.weight: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {"weight": TensorSpec((self.size,), role="gain", init="ones_normal")}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.weight = tensors["weight"]

    def forward(self, x: torch.Tensor, delta: Optional[torch.Tensor] = None,
                rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        n = x.shape[0] if rows is None else rows.shape[0]
        out = torch.empty((n, self.size), dtype=self.env.dtype, device=x.device)
        self.env.lib.add_rmsnorm(x, delta, self.weight, self.eps, rows, out)
        return out


register_norm("rmsnorm", RMSNorm)
