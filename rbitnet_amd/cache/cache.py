"""The cache of the engine: storage on the GPU, bookkeeping on the host.

* One slot per sequence (`alloc_slot` / `free_slot`): its length, its pages, its state.
* Keys and values per layer, in pages of 64 positions: K and V of a storage group are
  [layers of the group, pages, kv heads, 64, head_dim], so the 64 x head_dim tile of
  one head is contiguous.  The reference keeps one flat [position, kv head, dim] buffer
  per layer for its single sequence (crates/bitnet-core/src/llama/model.rs:29-42).
* Layers with equal needs (kv heads, head size, window) form a group with storage and
  a page pool of its own; a windowed group gives pages back as a sequence moves on.
* Fixed-size state per sequence: [layers of the group, slots, *shape], set to its
  initial value when the slot is handed out.  The Llama decoder has none; a mixer
  that asks for it gets it.
* Nothing is cleared when a slot or a page is reused: only positions below a
  sequence's length are ever read (the reference zero-fills, model.rs:44-51, without
  needing to: it reads 0..=pos only, :266,279).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from ..errors import CacheError, InferenceError
from ..parts.base import CacheRequest
from .pages import PAGE_SIZE, FreeList, PageTable, pages_for


@dataclass
class LayerCacheView:
    """What one layer's mixer sees of the cache during a step."""
    k_pages: Optional[torch.Tensor] = None        # [pages, kv heads, 64, head_dim]
    v_pages: Optional[torch.Tensor] = None
    block_table: Optional[torch.Tensor] = None    # int32 [B, pages per sequence], this step's sequences
    state: Optional[torch.Tensor] = None          # [slots, *shape]; index with ctx.slots


class KvGroup:
    def __init__(self, request: CacheRequest, layers: List[int], n_pages: int, dtype, device):
        self.request = request
        self.layers = list(layers)
        self.index = {l: i for i, l in enumerate(self.layers)}
        self.table = PageTable(n_pages, request.window)
        shape = (len(self.layers), n_pages, request.heads, PAGE_SIZE, request.head_dim)
        self.k = torch.empty(shape, dtype=dtype, device=device)
        self.v = torch.empty(shape, dtype=dtype, device=device)

    def bytes(self) -> int:
        return 2 * self.k.numel() * self.k.element_size()


class StateGroup:
    def __init__(self, request: CacheRequest, layers: List[int], n_slots: int, device):
        self.request = request
        self.layers = list(layers)
        self.index = {l: i for i, l in enumerate(self.layers)}
        shape = (len(self.layers), n_slots) + tuple(request.state_shape)
        self.data = torch.full(shape, request.state_init, dtype=request.state_dtype, device=device)

    def reset(self, slot: int) -> None:
        self.data[:, slot] = self.request.state_init


class Cache:
    def __init__(self, requests: Sequence[Optional[CacheRequest]], n_slots: int, max_tokens: int,
                 dtype: torch.dtype, device, readers: Optional[Dict[int, int]] = None):
        """requests[l]: what the mixer at place l of the schedule asked for (None: nothing);
        "layer" below means such a place.  readers[l] = j: place l reads place j's keys and
        values.  max_tokens: positions the pages of each
        group hold together, every sequence rounded up to whole pages."""
        if n_slots <= 0:
            raise CacheError("the cache needs at least one slot")
        self.n_slots = int(n_slots)
        self.n_pages = max(1, pages_for(int(max_tokens)))
        self.dtype = dtype
        self.device = device
        self.slots = FreeList(self.n_slots, "slot")
        self.lens: Dict[int, int] = {}
        self.kv_groups: List[KvGroup] = []
        self.state_groups: List[StateGroup] = []
        self.layer_kv: Dict[int, Tuple[KvGroup, int]] = {}
        self.layer_state: Dict[int, Tuple[StateGroup, int]] = {}
        by_key: Dict[Tuple, List[int]] = {}
        reqs: Dict[Tuple, CacheRequest] = {}
        for l, r in enumerate(requests):
            if r is None:
                continue
            if r.kind not in ("kv", "state"):
                raise CacheError(f"layer {l} asks for an unknown kind of cache {r.kind!r}")
            by_key.setdefault(r.key(), []).append(l)
            reqs[r.key()] = r
        for key, layers in by_key.items():
            r = reqs[key]
            if r.kind == "kv":
                g = KvGroup(r, layers, self.n_pages, dtype, device)
                self.kv_groups.append(g)
                for l in layers:
                    self.layer_kv[l] = (g, g.index[l])
            else:
                s = StateGroup(r, layers, self.n_slots, device)
                self.state_groups.append(s)
                for l in layers:
                    self.layer_state[l] = (s, s.index[l])
        for l, j in (readers or {}).items():
            if j not in self.layer_kv:
                raise CacheError(f"layer {l} reads the cache of layer {j}, which keeps none")
            self.layer_kv[l] = self.layer_kv[j]

    # ------------------------------------------------------------------ slots
    def alloc_slot(self) -> int:
        slot = self.slots.take()
        self.lens[slot] = 0
        for g in self.kv_groups:
            g.table.open(slot)
        for s in self.state_groups:
            s.reset(slot)
        return slot

    def free_slot(self, slot: int) -> None:
        self.slots.give_back(slot)
        del self.lens[slot]
        for g in self.kv_groups:
            g.table.close(slot)

    def length(self, slot: int) -> int:
        if slot not in self.lens:
            raise CacheError(f"slot {slot} is not in use")
        return self.lens[slot]

    @property
    def live_slots(self) -> List[int]:
        return self.slots.held()

    # ------------------------------------------------------------------ steps
    def reserve(self, slots: Sequence[int], q_lens: Sequence[int]) -> None:
        """Pages for the tokens a step is about to write.  All or nothing."""
        if len(set(slots)) != len(slots):
            raise InferenceError("a slot appears twice in one step")
        for slot in slots:
            self.length(slot)
        for g in self.kv_groups:
            need = sum(max(0, pages_for(self.lens[s] + q) - len(g.table.pages(s))) for s, q in zip(slots, q_lens))
            if need > g.table.pool.n_free:
                raise CacheError(
                    f"cache full: the step needs {need} more pages of {PAGE_SIZE} tokens, "
                    f"{g.table.pool.n_free} of {g.table.pool.n} are free")
        for g in self.kv_groups:
            for s, q in zip(slots, q_lens):
                g.table.ensure(s, self.lens[s] + q)

    def commit(self, slots: Sequence[int], q_lens: Sequence[int]) -> None:
        """The step has run: lengths grow, windowed groups give dead pages back."""
        for s, q in zip(slots, q_lens):
            self.lens[s] += q
            for g in self.kv_groups:
                g.table.release_behind(s, self.lens[s])

    def block_table(self, group: KvGroup, slots: Sequence[int], width: Optional[int] = None) -> List[List[int]]:
        rows = [group.table.pages(s) for s in slots]
        w = width or max(1, max(len(r) for r in rows))
        return [[(p if p >= 0 else 0) for p in r] + [0] * (w - len(r)) for r in rows]

    def view(self, layer: int, block_tables: Dict[int, torch.Tensor]) -> LayerCacheView:
        v = LayerCacheView()
        if layer in self.layer_kv:
            g, i = self.layer_kv[layer]
            v.k_pages, v.v_pages = g.k[i], g.v[i]
            v.block_table = block_tables[id(g)]
        if layer in self.layer_state:
            s, i = self.layer_state[layer]
            v.state = s.data[i]
        return v

    def check(self) -> None:
        self.slots.check()
        if set(self.lens) != set(self.slots.held()):
            raise CacheError("slots with a length and slots marked held differ")
        for g in self.kv_groups:
            g.table.check()
            if set(g.table.tables) != set(self.lens):
                raise CacheError("a page table exists for a slot that is not in use, or is missing")

    def bytes(self) -> int:
        return sum(g.bytes() for g in self.kv_groups) + sum(
            s.data.numel() * s.data.element_size() for s in self.state_groups)
