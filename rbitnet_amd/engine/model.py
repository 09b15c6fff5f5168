"""A model put together from a `ModelSpec`: embedding table, blocks, final norm, output
matrix.  Nothing here knows an architecture: the spec says which parts and which tensor
names, the part registries supply the parts.

The forward pass of one step follows the reference's per-token order
(crates/bitnet-core/src/llama/model.rs:229-315): embedding row, the layers in schedule
order, final norm and output matrix -- the last two only on the rows whose logits were
asked for.
"""
from __future__ import annotations

from typing import Callable, Dict, List, Optional

import torch

from ..config.spec import ModelSpec
from ..errors import ConfigError
from ..parts.base import BuildEnv, CacheRequest, TensorSpec, build_part
from ..parts.block import normed_for
from ..parts.linear import linear, pack_rows


def _build_blocks(spec: ModelSpec, env_for: Callable[[int], BuildEnv]):
    from ..parts.base import _REGISTRIES
    blocks = []
    for i, layer in enumerate(spec.layers):
        table = _REGISTRIES["block"]
        if layer.block not in table:
            raise ConfigError(f"unknown block kind {layer.block!r}; registered: {', '.join(sorted(table))}")
        blocks.append(table[layer.block](layer, env_for(i)))
    return blocks


def _named_parts(spec: ModelSpec, blocks, final_norm) -> Dict[str, object]:
    """prefix -> part, for every part that owns tensors."""
    out: Dict[str, object] = {}
    for layer, block in zip(spec.layers, blocks):
        for segment, part in block.parts().items():
            out[f"{layer.prefix}.{segment}"] = part
    return out


def expected_tensors(spec: ModelSpec) -> Dict[str, TensorSpec]:
    """Every tensor the model's parts declare, by full name, without touching a GPU."""
    env = BuildEnv(hidden_size=spec.hidden_size, dtype=torch.float32, device=torch.device("cpu"), lib=None)
    blocks = _build_blocks(spec, lambda i: env)
    final_norm = build_part("norm", spec.final_norm, env)
    out: Dict[str, TensorSpec] = {
        spec.embedding_name: TensorSpec((spec.vocab_size, spec.hidden_size)),
    }
    for prefix, part in _named_parts(spec, blocks, final_norm).items():
        for name, ts in part.tensor_specs().items():
            out[f"{prefix}.{name}"] = ts
    norm_specs = final_norm.tensor_specs()
    if len(norm_specs) == 1:
        out[spec.final_norm_name] = next(iter(norm_specs.values()))
    else:
        base = spec.final_norm_name.rsplit(".", 1)[0]
        for name, ts in norm_specs.items():
            out[f"{base}.{name}"] = ts
    if spec.head_name is not None:
        out[spec.head_name] = TensorSpec((spec.vocab_size, spec.hidden_size))
    return out


class Model:
    takes_gained_rows = True      # the output product takes what the last product left for the final norm

    def __init__(self, spec: ModelSpec, dtype: torch.dtype, device, lib, generic_only: bool = False,
                 max_seq_len: Optional[int] = None):
        if dtype not in (torch.float32, torch.bfloat16):
            raise ConfigError(f"compute dtype must be float32 or bfloat16, not {dtype}")
        self.spec = spec
        self.dtype = dtype
        self.device = torch.device(device)
        self.lib = lib
        self.generic_only = generic_only

        shared: Dict = {}

        def env_for(i: int) -> BuildEnv:
            env = BuildEnv(hidden_size=spec.hidden_size, dtype=dtype, device=self.device, lib=lib, layer_index=i,
                           shared=shared)
            env.generic_only = generic_only
            env.max_seq_len = max_seq_len         # tables keyed by position need no more rows than this
            return env

        self.blocks = _build_blocks(spec, env_for)
        self.final_norm = build_part("norm", spec.final_norm, env_for(-1))
        self.embedding: Optional[torch.Tensor] = None
        self.head: Optional[torch.Tensor] = None
        self.expected = expected_tensors(spec)

    # ------------------------------------------------------------------ cache needs
    def cache_requests(self) -> List[Optional[CacheRequest]]:
        """One entry per place in the schedule: a layer that runs twice keeps two caches,
        since its second run sees other inputs than its first."""
        out = []
        for i in self.spec.schedule:
            req = getattr(self.blocks[i].mixer, "cache_request", None)
            out.append(req() if req else None)
        return out

    def cache_readers(self) -> Dict[int, int]:
        """place in the schedule -> the place whose keys and values it reads: the latest
        earlier run of the layer that its mixer's `cache_from` names."""
        out = {}
        for place, i in enumerate(self.spec.schedule):
            j = getattr(self.blocks[i].mixer, "cache_from", None)
            if j is None:
                continue
            earlier = [p for p in range(place) if self.spec.schedule[p] == int(j)]
            if not earlier:
                raise ConfigError(f"layer {i} reads the cache of layer {j}, which does not run before it")
            out[place] = earlier[-1]
            own = getattr(self.blocks[i].mixer, "window", None)
            theirs = getattr(self.blocks[int(j)].mixer, "window", None)
            if theirs is not None and (own is None or int(own) > int(theirs)):
                raise ConfigError(
                    f"layer {i} looks back {own or 'without limit'} but reads the cache of layer {j}, "
                    f"which keeps only the last {theirs} positions")
        return out

    @property
    def graph_safe(self) -> bool:
        return (all(getattr(b, "graph_safe", False) for b in self.blocks)
                and getattr(self.final_norm, "graph_safe", False))

    def max_positions(self) -> int:
        return self.spec.max_positions

    # ------------------------------------------------------------------ weights
    def _place(self, t: torch.Tensor, ts: TensorSpec) -> torch.Tensor:
        """The tensor on the GPU in the dtype its role asks for; a change of the floating type
        is done there by the library's own copy kernel."""
        if ts.role == "table":
            return t.to(device=self.device, dtype=torch.int32).contiguous()
        want = torch.float32 if ts.role == "gain" else self.dtype
        t = t.to(device=self.device).contiguous()
        if t.dtype == want:
            return t
        if t.dtype not in (torch.float32, torch.bfloat16):
            return t.to(want)
        out = torch.empty(t.shape, dtype=want, device=self.device)
        if t.numel():
            width = t.shape[-1] if t.dim() >= 1 else 1
            self.lib.place_rows(t.reshape(-1, width), out.view(-1, width))
        return out

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        """tensors: full name -> tensor (any device, stored dtype).  Each is moved to the
        GPU in the dtype its role asks for and handed to its part."""
        spec = self.spec
        placed = lambda name: self._place(tensors[name], self.expected[name])
        self.embedding = placed(spec.embedding_name)
        if spec.head_name is None:
            self.head = self.embedding            # tied: the table's rows are also read one by one
        else:
            head = placed(spec.head_name)
            self.head = pack_rows(self.lib, [(head, 0, None, None)], head.shape[0], head.shape[1], head.dtype,
                                  head.device, not self.generic_only)
        for prefix, part in _named_parts(spec, self.blocks, self.final_norm).items():
            part.load({name: placed(f"{prefix}.{name}") for name in part.tensor_specs()})
        norm_specs = self.final_norm.tensor_specs()
        if len(norm_specs) == 1:
            self.final_norm.load({next(iter(norm_specs)): placed(spec.final_norm_name)})
        else:
            base = spec.final_norm_name.rsplit(".", 1)[0]
            self.final_norm.load({name: placed(f"{base}.{name}") for name in norm_specs})

    def weight_bytes(self) -> int:
        """Bytes of every weight a step reads once (a tied head counts once more: it is
        read again as the output matrix)."""
        total = 0
        for name, ts in self.expected.items():
            n = 1
            for s in ts.shape:
                n *= s
            if name == self.spec.embedding_name:
                continue          # the gather reads a few rows only
            total += n * (4 if ts.role in ("gain", "table") or self.dtype == torch.float32 else 2)
        if self.spec.head_name is None:
            total += self.spec.vocab_size * self.spec.hidden_size * (4 if self.dtype == torch.float32 else 2)
        return total

    # ------------------------------------------------------------------ forward
    def forward(self, ctx, cache, rows: torch.Tensor) -> torch.Tensor:
        """ctx.token_ids [T] -> float32 logits [len(rows), V] at the packed rows `rows`."""
        x = torch.empty((ctx.n_tokens, self.spec.hidden_size), dtype=torch.float32, device=self.device)
        self.lib.embed_gather(self.embedding, ctx.token_ids, x)
        pending = None
        schedule = self.spec.schedule
        for place, i in enumerate(schedule):
            block = self.blocks[i]
            view = cache.view(place, ctx.block_tables)
            if getattr(block, "takes_next_norm", False):
                after = self.blocks[schedule[place + 1]] if place + 1 < len(schedule) else None
                next_norm = self.final_norm if after is None else getattr(after, "first_norm", None)
                pending = block.forward(x, pending, ctx, view, next_norm=next_norm)
            else:
                pending = block.forward(x, pending, ctx, view)
        xn = normed_for(self, self.final_norm, x, pending, rows)
        return linear(self.lib, xn, self.head, torch.float32)
