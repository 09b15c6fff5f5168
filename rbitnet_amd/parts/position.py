"""Position encodings.  A position part turns the projected q, k, v of a step into the
rotated q and writes k and v into the cache, keyed by each token's absolute position.

Interface: encode_and_store(qkv, q_out, k_pages, v_pages, ctx, block_table,
                            n_heads, n_kv_heads, head_dim)
Optional:  rotation_tables() -> (cos, sin, style) when the encoding is a per-position,
           per-pair rotation; a mixer may then apply it inside a fused kernel.
           takes_terms = True: qkv may also be [P, T, W], the sums of the K slices of the
           product that made it, which encode_and_store adds up in their order as it reads.

"rope": the rotation of the reference (crates/bitnet-core/src/llama/model.rs:122-136):
inv_i = 1 / theta^(2i/D), angle = pos * inv_i, pairs (x[2i], x[2i+1]) ("interleaved") or
(x[i], x[i+D/2]) ("half").  The angle table [positions, D/2] is computed once on the
host in float64 and held as float32 cosines and sines; this is the one place where
frequency scaling rules live.  Any per-position, per-pair rotation can be expressed by
another table, so a new rule needs a new table builder only.
"none": no rotation; k and v are stored as they are.
"""
from __future__ import annotations

import math
from typing import Dict, Optional

import torch

from ..errors import ConfigError
from .base import BuildEnv, Part, register_position


def rope_inverse_frequencies(head_dim: int, theta: float, scaling: Optional[Dict]) -> torch.Tensor:
    """float64 [D/2].  `scaling` None or {"rope_type": "llama3", factor, low_freq_factor,
    high_freq_factor, original_max_position_embeddings}: wavelengths shorter than
    original/high keep their frequency, longer than original/low have it divided by
    factor, and those between are blended linearly in original/wavelength."""
    i = torch.arange(head_dim // 2, dtype=torch.float64)
    inv = torch.pow(torch.tensor(float(theta), dtype=torch.float64), -2.0 * i / head_dim)
    if not scaling:
        return inv
    kind = scaling.get("rope_type", "default")
    if kind == "default":
        return inv
    if kind != "llama3":
        raise ConfigError(f"unsupported rope scaling {kind!r}")
    factor = float(scaling["factor"])
    low = float(scaling["low_freq_factor"])
    high = float(scaling["high_freq_factor"])
    orig = float(scaling["original_max_position_embeddings"])
    wavelength = 2.0 * math.pi / inv
    blend = (orig / wavelength - low) / (high - low)
    mixed = (1.0 - blend) * inv / factor + blend * inv
    out = torch.where(wavelength > orig / low, inv / factor, mixed)
    out = torch.where(wavelength < orig / high, inv, out)
    return out


class Rope(Part):
    graph_safe = True
    plan_safe = True
    takes_terms = True      # qkv may come as [P, T, W]: terms that the kernel adds up

    def __init__(self, params: Dict, env: BuildEnv):
        self.head_dim = int(params["head_dim"])
        self.style = {"interleaved": 0, "half": 1}.get(params.get("style", "interleaved"))
        if self.style is None:
            raise ConfigError(f"unknown rope style {params.get('style')!r}")
        self.max_positions = int(params["max_positions"])
        if getattr(env, "max_seq_len", None):
            self.max_positions = min(self.max_positions, int(env.max_seq_len))
        self.env = env
        inv = rope_inverse_frequencies(self.head_dim, float(params["theta"]), params.get("scaling"))
        self.inv_freq = inv
        self.cos: Optional[torch.Tensor] = None
        self.sin: Optional[torch.Tensor] = None
        if env.lib is not None:
            # one table for all layers with the same rotation: a step's row is then fetched
            # from memory once and found in cache by the layers after the first
            key = ("rope", self.head_dim, float(params["theta"]), repr(sorted((params.get("scaling") or {}).items())),
                   self.max_positions, str(env.device))
            if key not in env.shared:
                angles = torch.arange(self.max_positions, dtype=torch.float64)[:, None] * inv[None, :]
                env.shared[key] = (torch.cos(angles).to(torch.float32).to(env.device).contiguous(),
                                   torch.sin(angles).to(torch.float32).to(env.device).contiguous())
            self.cos, self.sin = env.shared[key]

    def rotation_tables(self):
        """(cos, sin, pairing style): lets a mixer fold the rotation into its own kernel."""
        return self.cos, self.sin, self.style

    def encode_and_store(self, qkv, q_out, k_pages, v_pages, ctx, block_table, n_heads, n_kv, head_dim) -> None:
        self.env.lib.rope_kv_write(qkv, self.cos, self.sin, self.style, q_out, k_pages, v_pages, ctx.tok_pos,
                                   ctx.tok_seq, block_table, n_heads, n_kv, head_dim)


class NoPosition(Part):
    graph_safe = True
    plan_safe = True
    takes_terms = True

    def __init__(self, params: Dict, env: BuildEnv):
        self.env = env
        self.max_positions = int(params.get("max_positions", 1 << 30))

    def rotation_tables(self):
        return None, None, 0

    def encode_and_store(self, qkv, q_out, k_pages, v_pages, ctx, block_table, n_heads, n_kv, head_dim) -> None:
        self.env.lib.rope_kv_write(qkv, None, None, 0, q_out, k_pages, v_pages, ctx.tok_pos, ctx.tok_seq,
                                   block_table, n_heads, n_kv, head_dim)


register_position("rope", Rope)
register_position("none", NoPosition)
