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
* One page and one slot more than are ever handed out, the spare ones: a captured decode
  step made for more sequences than are running fills its idle rows with a sequence of
  length 0 in the spare slot, whose keys, values and state go to the spare page and the
  spare state and nowhere else.

A storage group is a class registered under the kind of a `CacheRequest`
(`register_cache_kind`), built as `cls(request, layers, n_pages, n_slots, dtype, device)`:

    kind                  the request kind it serves
    open(slot), close(slot)
    fill_view(view, i, block_tables)     what layer i of the group shows a mixer in a step
    bytes()                              its storage
    bytes_per_token(request, n_layers, dtype)      static: growth per token of a sequence

and, when it grows with its sequences in pages (`paged = True`; derive from `PagedGroup`):

    table                 a `PageTable` (ensure, release_behind, pages, pool)
    pages_missing(slot, n_tokens)
    spare_page            index of the page that idle rows write to (its storage holds
                          n_pages + 1 pages)

A group that keeps something per slot gives it room for n_slots + 1 slots.  Only a "kv"
group can be read by another layer (`readers`): what is shared are keys and values.
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


class PagedGroup:
    """What the cache needs of a group that grows with its sequences in pages: a page table
    over n_pages pages, and one page more that is never handed out."""
    paged = True

    def __init__(self, request: CacheRequest, layers: List[int], n_pages: int):
        self.request = request
        self.layers = list(layers)
        self.index = {l: i for i, l in enumerate(self.layers)}
        self.table = PageTable(n_pages, request.window)
        self.spare_page = int(n_pages)

    def open(self, slot: int) -> None:
        self.table.open(slot)

    def close(self, slot: int) -> None:
        self.table.close(slot)

    def pages_missing(self, slot: int, n_tokens: int) -> int:
        return max(0, pages_for(n_tokens) - len(self.table.pages(slot)))


class KvGroup(PagedGroup):
    """Keys and values per token in pages; a window gives pages back as a sequence moves on."""
    kind = "kv"

    def __init__(self, request: CacheRequest, layers: List[int], n_pages: int, n_slots: int, dtype, device):
        super().__init__(request, layers, n_pages)
        shape = (len(self.layers), n_pages + 1, request.heads, PAGE_SIZE, request.head_dim)
        self.k = torch.empty(shape, dtype=dtype, device=device)
        self.v = torch.empty(shape, dtype=dtype, device=device)

    @staticmethod
    def bytes_per_token(request: CacheRequest, n_layers: int, dtype: torch.dtype) -> int:
        return 2 * n_layers * request.heads * request.head_dim * torch.empty((), dtype=dtype).element_size()

    def fill_view(self, view: "LayerCacheView", i: int, block_tables: Dict[int, torch.Tensor]) -> None:
        view.k_pages, view.v_pages = self.k[i], self.v[i]
        view.block_table = block_tables[id(self)]

    def bytes(self) -> int:
        return 2 * self.k.numel() * self.k.element_size()


class StateGroup:
    """A fixed number of values per sequence, set to their initial value when a slot is handed out."""
    kind = "state"

    def __init__(self, request: CacheRequest, layers: List[int], n_pages: int, n_slots: int, dtype, device):
        self.request = request
        self.layers = list(layers)
        self.index = {l: i for i, l in enumerate(self.layers)}
        shape = (len(self.layers), n_slots + 1) + tuple(request.state_shape)        # the last: the spare slot's
        self.data = torch.full(shape, request.state_init, dtype=request.state_dtype, device=device)

    @staticmethod
    def bytes_per_token(request: CacheRequest, n_layers: int, dtype: torch.dtype) -> int:
        return 0

    def open(self, slot: int) -> None:
        self.data[:, slot] = self.request.state_init

    def close(self, slot: int) -> None:
        pass

    def fill_view(self, view: "LayerCacheView", i: int, block_tables: Dict[int, torch.Tensor]) -> None:
        view.state = self.data[i]

    def bytes(self) -> int:
        return self.data.numel() * self.data.element_size()


# kind of a CacheRequest -> the class that stores it (the interface: see the module's text)
_GROUP_KINDS: Dict[str, type] = {"kv": KvGroup, "state": StateGroup}


def register_cache_kind(kind: str, group_class: type) -> None:
    _GROUP_KINDS[kind] = group_class


def bytes_per_token(requests: Sequence[Optional[CacheRequest]], dtype: torch.dtype) -> int:
    """Bytes that one more token of one sequence adds over all layers."""
    counts: Dict[Tuple, int] = {}
    reqs: Dict[Tuple, CacheRequest] = {}
    for r in requests:
        if r is not None and r.kind in _GROUP_KINDS:
            counts[r.key()] = counts.get(r.key(), 0) + 1
            reqs[r.key()] = r
    return sum(_GROUP_KINDS[reqs[k].kind].bytes_per_token(reqs[k], n, dtype) for k, n in counts.items())


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
        self.spare_slot = self.n_slots          # never handed out: where idle rows of a captured step live
        self.n_pages = max(1, pages_for(int(max_tokens)))
        self.dtype = dtype
        self.device = device
        self.slots = FreeList(self.n_slots, "slot")
        self.lens: Dict[int, int] = {}
        self.groups: List = []
        self.layer_groups: Dict[int, List[Tuple[object, int]]] = {}
        by_key: Dict[Tuple, List[int]] = {}
        reqs: Dict[Tuple, CacheRequest] = {}
        for l, r in enumerate(requests):
            if r is None:
                continue
            if r.kind not in _GROUP_KINDS:
                raise CacheError(f"layer {l} asks for an unknown kind of cache {r.kind!r} "
                                 f"(known: {', '.join(sorted(_GROUP_KINDS))})")
            by_key.setdefault(r.key(), []).append(l)
            reqs[r.key()] = r
        for key, layers in by_key.items():
            r = reqs[key]
            g = _GROUP_KINDS[r.kind](r, layers, self.n_pages, self.n_slots, dtype, device)
            self.groups.append(g)
            for l in layers:
                self.layer_groups.setdefault(l, []).append((g, g.index[l]))
        for l, j in (readers or {}).items():
            theirs = [(g, i) for g, i in self.layer_groups.get(j, []) if g.kind == "kv"]
            if not theirs:
                raise CacheError(f"layer {l} reads the cache of layer {j}, which keeps none")
            self.layer_groups.setdefault(l, []).extend(theirs)

    @property
    def kv_groups(self) -> List:
        """The groups that grow with their sequences in pages."""
        return [g for g in self.groups if getattr(g, "paged", False)]

    @property
    def state_groups(self) -> List:
        return [g for g in self.groups if g.kind == "state"]

    # ------------------------------------------------------------------ slots
    def alloc_slot(self) -> int:
        slot = self.slots.take()
        self.lens[slot] = 0
        for g in self.groups:
            g.open(slot)
        return slot

    def free_slot(self, slot: int) -> None:
        self.slots.give_back(slot)
        del self.lens[slot]
        for g in self.groups:
            g.close(slot)

    def length(self, slot: int) -> int:
        if slot not in self.lens:
            raise CacheError(f"slot {slot} is not in use")
        return self.lens[slot]

    @property
    def live_slots(self) -> List[int]:
        return self.slots.held()

    # ------------------------------------------------------------------ room, in tokens
    def token_capacity(self) -> int:
        """The most tokens all live sequences can hold together, each counted with
        `tokens_needed` of its length."""
        return min((g.table.pool.n * PAGE_SIZE for g in self.kv_groups), default=1 << 40)

    @staticmethod
    def tokens_needed(n_tokens: int) -> int:
        """What a sequence of n tokens takes of the capacity: whole pages."""
        return pages_for(n_tokens) * PAGE_SIZE

    def can_grow(self, slot: int, by: int = 1) -> bool:
        """Whether the sequence can hold `by` more tokens: in the pages it has, or in free ones."""
        n = self.length(slot) + by
        return all(g.pages_missing(slot, n) <= g.table.pool.n_free for g in self.kv_groups)

    @staticmethod
    def pages_per_sequence(n_tokens: int) -> int:
        return pages_for(n_tokens)

    # ------------------------------------------------------------------ steps
    def reserve(self, slots: Sequence[int], q_lens: Sequence[int]) -> None:
        """Pages for the tokens a step is about to write.  All or nothing."""
        if len(set(slots)) != len(slots):
            raise InferenceError("a slot appears twice in one step")
        for slot in slots:
            self.length(slot)
        for g in self.kv_groups:
            need = sum(g.pages_missing(s, self.lens[s] + q) for s, q in zip(slots, q_lens))
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

    def group_keys(self) -> List[int]:
        return [id(g) for g in self.kv_groups]

    def block_tables(self, slots: Sequence[int]) -> Dict[int, List[List[int]]]:
        """Per paged group, per sequence of the step, its pages (a page given back behind a
        window is never read; 0 stands in for it).  The spare slot holds the spare page."""
        return {id(g): [[g.spare_page] if s == self.spare_slot else [(p if p >= 0 else 0) for p in g.table.pages(s)]
                        for s in slots] for g in self.kv_groups}

    def view(self, layer: int, block_tables: Dict[int, torch.Tensor]) -> LayerCacheView:
        v = LayerCacheView()
        for g, i in self.layer_groups.get(layer, []):
            g.fill_view(v, i, block_tables)
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
        return sum(g.bytes() for g in self.groups)
