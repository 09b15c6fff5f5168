"""The cache's bookkeeping on the host (CPU tensors stand in for the GPU storage): no
slot or page lost, held twice or freed twice; groups; windows; fixed-size state."""
import random

import pytest
import torch

from rbitnet_amd.cache import PAGE_SIZE, Cache, FreeList, pages_for
from rbitnet_amd.errors import CacheError, InferenceError
from rbitnet_amd.parts.base import CacheRequest


def test_free_list_hands_out_lowest_first_and_refuses_misuse():
    f = FreeList(3, "slot")
    assert [f.take(), f.take(), f.take()] == [0, 1, 2]
    with pytest.raises(CacheError, match="no free slot"):
        f.take()
    f.give_back(1)
    with pytest.raises(CacheError, match="freed twice"):
        f.give_back(1)
    with pytest.raises(CacheError, match="does not exist"):
        f.give_back(7)
    assert f.take() == 1
    f.check()


def _cache(n_slots=4, max_tokens=64 * 10, window=None, layers=3):
    reqs = [CacheRequest("kv", heads=2, head_dim=8, window=window) for _ in range(layers)]
    return Cache(reqs, n_slots, max_tokens, torch.float32, "cpu")


def test_pages_follow_lengths_and_come_back():
    c = _cache()
    assert c.n_pages == 10 and len(c.kv_groups) == 1
    g = c.kv_groups[0]
    assert g.k.shape == (3, 10 + 1, 2, PAGE_SIZE, 8)           # and the spare page
    a, b = c.alloc_slot(), c.alloc_slot()
    c.reserve([a, b], [65, 1])
    assert len(g.table.pages(a)) == 2 and len(g.table.pages(b)) == 1
    c.commit([a, b], [65, 1])
    assert c.length(a) == 65 and c.length(b) == 1
    c.reserve([a, b], [1, 1])                      # no new page: 66 <= 128, 2 <= 64
    assert g.table.pool.n_held == 3
    c.commit([a, b], [1, 1])
    c.check()
    c.free_slot(a)
    assert g.table.pool.n_held == 1
    with pytest.raises(CacheError):
        c.free_slot(a)
    with pytest.raises(CacheError, match="not in use"):
        c.length(a)
    a2 = c.alloc_slot()
    assert a2 == a and c.length(a2) == 0           # the slot is used again, empty
    c.check()


def test_reserve_is_all_or_nothing():
    c = _cache(max_tokens=64 * 4)
    a, b = c.alloc_slot(), c.alloc_slot()
    c.reserve([a], [64 * 3])
    c.commit([a], [64 * 3])
    with pytest.raises(CacheError, match="cache full"):
        c.reserve([a, b], [1, 65])                 # needs 1 + 2 pages, 1 is free
    assert c.kv_groups[0].table.pool.n_held == 3   # nothing was taken
    c.check()
    with pytest.raises(InferenceError, match="twice"):
        c.reserve([a, a], [1, 1])


def test_random_traffic_never_loses_anything():
    rng = random.Random(5)
    c = _cache(n_slots=6, max_tokens=64 * 40)
    live = {}
    for _ in range(2000):
        op = rng.random()
        if op < 0.3 and len(live) < 6:
            live[c.alloc_slot()] = 0
        elif op < 0.5 and live:
            s = rng.choice(list(live))
            c.free_slot(s)
            del live[s]
        elif live:
            s = rng.choice(list(live))
            q = rng.choice([1, 1, 1, 7, 64, 100])
            try:
                c.reserve([s], [q])
                c.commit([s], [q])
                live[s] += q
            except CacheError:
                pass
        c.check()
        g = c.kv_groups[0]
        assert g.table.pool.n_held == sum(pages_for(n) for n in live.values())
        assert {s: c.length(s) for s in live} == live
    for s in list(live):
        c.free_slot(s)
    c.check()
    assert c.kv_groups[0].table.pool.n_free == 40 and c.slots.n_free == 6


def test_groups_by_need_and_readers():
    reqs = [CacheRequest("kv", heads=2, head_dim=8), CacheRequest("kv", heads=2, head_dim=8, window=100),
            None, CacheRequest("kv", heads=2, head_dim=8), CacheRequest("kv", heads=1, head_dim=16),
            CacheRequest("state", state_shape=(3, 2), state_init=1.5)]
    c = Cache(reqs, 2, 64 * 8, torch.float32, "cpu", readers={2: 1})
    assert len(c.kv_groups) == 3 and len(c.state_groups) == 1
    kv = lambda l: next((g, i) for g, i in c.layer_groups[l] if g.kind == "kv")
    full = kv(0)[0]
    assert full.layers == [0, 3] and kv(3) == (full, 1)
    assert kv(2) == kv(1)                            # layer 2 reads layer 1's keys and values
    assert kv(4)[0].k.shape == (1, 8 + 1, 1, PAGE_SIZE, 16)
    with pytest.raises(CacheError, match="keeps none"):
        Cache([None, CacheRequest("kv", heads=1, head_dim=8)], 1, 64, torch.float32, "cpu", readers={1: 0})


def test_window_gives_pages_back_early():
    c = _cache(max_tokens=64 * 6, window=70, layers=1)
    g = c.kv_groups[0]
    s = c.alloc_slot()
    c.reserve([s], [200])
    c.commit([s], [200])
    # keys below 200 - 70 + 1 = 131 are dead: pages 0 and 1 (positions < 128)
    assert g.table.pages(s)[:2] == [-1, -1] and g.table.pool.n_held == 2
    for _ in range(200):
        c.reserve([s], [1])
        c.commit([s], [1])
        c.check()
    assert c.length(s) == 400 and g.table.pool.n_held <= 3     # a full group would hold 7
    assert c.block_tables([s])[id(g)][0][0] == 0                   # dead entries read as a valid page id
    c.free_slot(s)
    assert g.table.pool.n_free == 6


def test_state_is_reset_when_a_slot_is_handed_out():
    reqs = [CacheRequest("state", state_shape=(4,), state_init=2.0)]
    c = Cache(reqs, 2, 64, torch.float32, "cpu")
    s = c.alloc_slot()
    st = c.view(0, {}).state
    assert st.shape == (2 + 1, 4) and torch.all(st[s] == 2.0)         # two slots and the spare one
    st[s] += 5
    c.free_slot(s)
    assert c.alloc_slot() == s and torch.all(c.view(0, {}).state[s] == 2.0)


def test_a_third_kind_of_group_registered_from_here():
    """A paged group of the test's own (one number per position and layer, shown to its mixer in a
    field of its own) beside the built-in kinds: reserved, committed, grown, freed and checked like them."""
    from rbitnet_amd.cache.cache import PagedGroup, register_cache_kind

    class MarksGroup(PagedGroup):
        kind = "marks"

        def __init__(self, request, layers, n_pages, n_slots, dtype, device):
            super().__init__(request, layers, n_pages)
            self.marks = torch.zeros((len(self.layers), n_pages + 1, PAGE_SIZE), dtype=dtype, device=device)

        @staticmethod
        def bytes_per_token(request, n_layers, dtype):
            return n_layers * torch.empty((), dtype=dtype).element_size()

        def fill_view(self, view, i, block_tables):
            view.marks = self.marks[i]
            view.marks_table = block_tables[id(self)]

        def bytes(self):
            return self.marks.numel() * self.marks.element_size()

    register_cache_kind("marks", MarksGroup)
    reqs = [CacheRequest("kv", heads=1, head_dim=4), CacheRequest("marks"), CacheRequest("marks")]
    c = Cache(reqs, 2, 64 * 3, torch.float32, "cpu")
    marks = next(g for g in c.groups if g.kind == "marks")
    assert marks in c.kv_groups and len(c.kv_groups) == 2 and marks.layers == [1, 2]
    assert c.token_capacity() == 64 * 3
    a, b = c.alloc_slot(), c.alloc_slot()
    c.reserve([a, b], [100, 5])
    c.commit([a, b], [100, 5])
    tables = c.block_tables([a, b, c.spare_slot])
    assert [len(t) for t in tables[id(marks)]] == [2, 1, 1] and tables[id(marks)][2] == [marks.spare_page]
    view = c.view(2, {id(g): torch.tensor([[0]]) for g in c.kv_groups})
    assert view.marks.shape == (3 + 1, PAGE_SIZE) and view.k_pages is None
    assert not c.can_grow(a, 64) and c.can_grow(b, 59) and not c.can_grow(b, 60)       # both groups have one page left
    with pytest.raises(CacheError, match="cache full"):
        c.reserve([a, b], [29, 60])
    c.check()
    c.free_slot(a)
    assert marks.table.pool.n_free == 2 and c.can_grow(b, 60)
    c.free_slot(b)
    c.check()
    with pytest.raises(CacheError, match="keeps none"):           # only keys and values can be read by another layer
        Cache([CacheRequest("marks"), None], 1, 64, torch.float32, "cpu", readers={1: 0})
