"""A model put together from a `ModelSpec`: an embedding, blocks, a head.  Nothing here knows
an architecture, and the forward pass holds no stage of its own: the spec says which parts and
which tensor names, the part registries supply the parts.

The forward pass of one step follows the reference's per-token order
(crates/bitnet-core/src/llama/model.rs:229-315): embedding row, the layers in schedule
order, final norm and output matrix -- the last two (the head) only on the rows whose logits
were asked for.
"""
from __future__ import annotations

from typing import Callable, Dict, List, Optional

import torch

from ..config.spec import ModelSpec
from ..errors import ConfigError
from ..parts.base import BuildEnv, CacheRequest, TensorSpec, build_part
from ..parts.stream import run_blocks


def _build_blocks(spec: ModelSpec, env_for: Callable[[int], BuildEnv]):
    from ..parts.base import _REGISTRIES
    blocks = []
    for i, layer in enumerate(spec.layers):
        table = _REGISTRIES["block"]
        if layer.block not in table:
            raise ConfigError(f"unknown block kind {layer.block!r}; registered: {', '.join(sorted(table))}")
        blocks.append(table[layer.block](layer, env_for(i)))
    return blocks


def _ends(spec: ModelSpec, env: BuildEnv):
    return build_part("embedding", spec.embedding, env), build_part("head", spec.head, env)


def _named_parts(spec: ModelSpec, blocks) -> Dict[str, object]:
    """prefix -> part, for every part of a block that owns tensors (the two ends name theirs in full)."""
    out: Dict[str, object] = {}
    for layer, block in zip(spec.layers, blocks):
        for segment, part in block.parts().items():
            out[f"{layer.prefix}.{segment}"] = part
    return out


def _expected(spec: ModelSpec, blocks, embedding, head) -> Dict[str, TensorSpec]:
    out: Dict[str, TensorSpec] = {}
    for part in (embedding, head):
        out.update(part.tensor_specs())
    for prefix, part in _named_parts(spec, blocks).items():
        for name, ts in part.tensor_specs().items():
            out[f"{prefix}.{name}"] = ts
    return out


def expected_tensors(spec: ModelSpec) -> Dict[str, TensorSpec]:
    """Every tensor the model's parts declare, by full name, without touching a GPU."""
    env = BuildEnv(hidden_size=spec.hidden_size, dtype=torch.float32, device=torch.device("cpu"), lib=None)
    blocks = _build_blocks(spec, lambda i: env)
    embedding, head = _ends(spec, env)
    return _expected(spec, blocks, embedding, head)


class Model:
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
        self.embedding, self.head = _ends(spec, env_for(-1))
        self.expected = _expected(spec, self.blocks, self.embedding, self.head)

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
        return all(getattr(p, "graph_safe", False) for p in list(self.blocks) + [self.embedding, self.head])

    @property
    def plan_safe(self) -> bool:
        """Whether every part's forward does nothing on the device but call the kernel library, so
        that a step's launches can be recorded there and issued again from C++."""
        return all(getattr(p, "plan_safe", False) for p in list(self.blocks) + [self.embedding, self.head])

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
        placed = lambda name: self._place(tensors[name], self.expected[name])
        self.embedding.load({name: placed(name) for name in self.embedding.tensor_specs()})
        self.head.load({name: placed(name) for name in self.head.tensor_specs()}, embedding=self.embedding)
        for prefix, part in _named_parts(self.spec, self.blocks).items():
            part.load({name: placed(f"{prefix}.{name}") for name in part.tensor_specs()})

    def weight_bytes(self) -> int:
        """Bytes of every weight a step reads once: all tensors of the blocks, and of the two ends
        what they say (`step_bytes`: a table that is only gathered from counts nothing, a matrix
        shared with it counts where it is read in full)."""
        esize = 4 if self.dtype == torch.float32 else 2
        total = 0
        for prefix, part in _named_parts(self.spec, self.blocks).items():
            total += _tensor_bytes(part.tensor_specs().values(), esize)
        for part in (self.embedding, self.head):
            own = getattr(part, "step_bytes", None)
            total += own(esize) if own else _tensor_bytes(part.tensor_specs().values(), esize)
        return total

    def activation_bytes(self, n_tokens: int, n_rows: int = 1) -> int:
        """About what a step of n_tokens tokens that asks for n_rows rows of logits allocates beside
        the weights and the cache (an estimate for sizing and for refusing a step early, not a bound)."""
        from ..engine.engine import ACTIVATION_ROWS_PER_TOKEN
        widest = self.spec.hidden_size
        for prefix, part in _named_parts(self.spec, self.blocks).items():
            for ts in part.tensor_specs().values():
                if ts.role == "matrix" and len(ts.shape) == 2:
                    widest = max(widest, int(ts.shape[0]))
        return 4 * (ACTIVATION_ROWS_PER_TOKEN * widest * int(n_tokens) + 2 * self.spec.vocab_size * int(n_rows))

    # ------------------------------------------------------------------ forward
    def forward(self, ctx, cache, rows: torch.Tensor) -> torch.Tensor:
        """ctx.token_ids [T] -> float32 logits [len(rows), V] at the packed rows `rows`."""
        x = self.embedding.forward(ctx)
        pending = run_blocks(self.blocks, self.spec.schedule, x, ctx, cache, getattr(self.head, "first_norm", None))
        return self.head.forward(x, pending, rows, ctx)


def _tensor_bytes(specs, element_size: int) -> int:
    total = 0
    for ts in specs:
        n = 1
        for s in ts.shape:
            n *= s
        total += n * (4 if ts.role in ("gain", "table") else element_size)
    return total
