"""Choosing the next token from float32 logits.

Reference (crates/bitnet-core/src/llama/runtime.rs:81-107): temperature <= 0 takes the
greatest logit (NaN counted as -inf); otherwise z = logits / T, e = exp(z - max z),
r = u * sum(e) with u uniform in [0, 1), and the first index whose running sum reaches r
wins, the last index if none does.  The reference has no top-k or top-p, so neither is
here.  Among equal maxima the lowest index is taken (the reference's iterator keeps
the last; for float32 logits of a real model the case does not arise).

The reference draws u from an unseeded thread generator (runtime.rs:62).  Here u comes
from a counter-based generator keyed by (seed, sequence id, number of tokens the
sequence has sampled), so a sequence draws the same numbers alone or in any batch.
"""
from __future__ import annotations

import hashlib
import struct
from typing import Optional, Sequence

import torch


def uniform(seed: int, sequence_id: int, n_sampled: int) -> float:
    """u in [0, 1) with 24 random bits (exactly representable in float32)."""
    digest = hashlib.blake2b(struct.pack("<qqq", int(seed), int(sequence_id), int(n_sampled)),
                             digest_size=8).digest()
    return (int.from_bytes(digest, "little") >> 40) / float(1 << 24)


class Sampler:
    """Samples one token per row of a logits matrix on the GPU."""

    def __init__(self, lib, device):
        self.lib = lib
        self.device = device

    def sample(self, logits: torch.Tensor, temperatures: Optional[Sequence[float]] = None,
               uniforms: Optional[Sequence[float]] = None) -> list:
        n = logits.shape[0]
        tokens = torch.empty(n, dtype=torch.int32, device=logits.device)
        if temperatures is None or all(t <= 0.0 for t in temperatures):
            self.lib.sample(logits, None, None, tokens)
        else:
            if uniforms is None or len(uniforms) != n or len(temperatures) != n:
                raise ValueError("temperature sampling needs one temperature and one uniform number per row")
            both = torch.tensor([list(temperatures), list(uniforms)], dtype=torch.float32).to(logits.device)
            self.lib.sample(logits, both[0].contiguous(), both[1].contiguous(), tokens)
        return tokens.tolist()
