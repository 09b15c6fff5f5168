"""The generation loop's decisions, with a scripted engine in place of the GPU."""
import pytest
import torch

from rbitnet_amd.cache import Cache
from rbitnet_amd.engine.generate import decide, generate, plan_batches
from rbitnet_amd.errors import InferenceError
from rbitnet_amd.parts.base import CacheRequest
from rbitnet_amd.sampling import uniform


class _Spec:
    stop_token_ids = [9]
    bos_token_id = None
    vocab_size = 16


class ScriptedEngine:
    """next token = (last token fed + 1) % 16, computed from what is fed; keeps a real
    cache bookkeeper so that slots and pages are accounted for."""

    def __init__(self, max_batch=2, max_tokens=64 * 8, max_seq_len=64):
        self.spec = _Spec()
        self.max_batch = max_batch
        self.max_seq_len = max_seq_len
        self.cache = Cache([CacheRequest("kv", heads=1, head_dim=2)], max_batch, max_tokens, torch.float32, "cpu")
        self.steps = []
        self.sampler = self

    def alloc_slot(self):
        return self.cache.alloc_slot()

    def free_slot(self, s):
        self.cache.free_slot(s)

    def step(self, entries, want):
        assert want == "last"
        slots = [s for s, _ in entries]
        q = [len(t) for _, t in entries]
        self.cache.reserve(slots, q)
        self.cache.commit(slots, q)
        self.steps.append([(s, list(t)) for s, t in entries])
        return [(t[-1] + 1) % 16 for _, t in entries]

    def sample(self, logits, temperatures=None, uniforms=None):
        return list(logits)

    def decode_step(self, slots, tokens, temperatures=None, uniforms=None):
        return self.sample(self.step([(s, [t]) for s, t in zip(slots, tokens)], "last"))


def test_decide():
    assert decide(9, 0, 10, 5, {9}) == "stop"
    assert decide(3, 9, 10, 5, {9}) == "length"
    assert decide(3, 0, 10, 0, {9}) == "context"
    assert decide(3, 0, 10, 5, {9}) is None
    assert decide(9, 9, 10, 0, {9}) == "stop"          # a stop token wins over the limits


def test_stop_token_is_not_emitted_and_not_fed():
    eng = ScriptedEngine()
    (r,) = generate(eng, [[5]], max_tokens=20, temperature=0.0)
    assert r.tokens == [6, 7, 8] and r.finish_reason == "stop"     # 9 ends it (runtime.rs:67-69)
    assert [e[0][1] for e in eng.steps] == [[5], [6], [7], [8]]    # 9 was never run
    assert eng.cache.slots.n_held == 0


def test_max_tokens_and_no_wasted_step():
    eng = ScriptedEngine()
    (r,) = generate(eng, [[10, 11]], max_tokens=3, temperature=0.0)
    assert r.tokens == [12, 13, 14] and r.finish_reason == "length"
    assert len(eng.steps) == 3                                      # the last token is not fed
    assert generate(eng, [[1]], max_tokens=0)[0].finish_reason == "length"


def test_a_limit_of_its_own_for_every_request():
    """max_tokens as a list: every request ends at its own limit, a request with none runs no step,
    and the cache is planned with each request's own growth."""
    eng = ScriptedEngine(max_batch=3)
    rs = generate(eng, [[10], [1], [12], [2]], max_tokens=[3, 0, 1, 5], temperature=0.0, stop_token_ids=[])
    assert [r.tokens for r in rs] == [[11, 12, 13], [], [13], [3, 4, 5, 6, 7]]
    assert [r.finish_reason for r in rs] == ["length"] * 4
    assert eng.steps[0] == [(0, [10]), (1, [12]), (2, [2])]          # the request without a budget holds no slot
    assert eng.steps[1] == [(0, [11]), (2, [3])]                      # the one with a single token has left
    assert [len(s) for s in eng.steps] == [3, 2, 2, 1, 1]
    with pytest.raises(InferenceError, match="values of max_tokens"):
        generate(eng, [[1], [2]], max_tokens=[3])
    assert plan_batches([10, 10, 10], [100, 20, 20], 8, 1000, 192, lambda n: (n + 63) // 64 * 64) == [[0, 1], [2]]
    assert eng.cache.slots.n_held == 0


def test_unequal_batch_shorter_requests_end_earlier_and_slots_are_reused():
    eng = ScriptedEngine(max_batch=2)
    prompts = [[7], [1, 2], [8], [0]]
    rs = generate(eng, prompts, max_tokens=4, temperature=0.0)
    assert [r.tokens for r in rs] == [[8], [3, 4, 5, 6], [], [1, 2, 3, 4]]
    assert [r.finish_reason for r in rs] == ["stop", "length", "stop", "length"]
    # first batch: both prompts in one step, then the survivor alone
    assert eng.steps[0] == [(0, [7]), (1, [1, 2])]
    assert eng.steps[1] == [(0, [8]), (1, [3])]
    assert eng.steps[2] == [(1, [4])]
    # second batch starts after the first is done, in the same slots
    second = [s for s in eng.steps if (0, [8]) in s and len(s) == 2 and s[1][1] == [0]]
    assert second, eng.steps
    assert eng.cache.slots.n_held == 0
    eng.cache.check()


def test_context_limit_ends_a_sequence_without_failing_the_batch():
    eng = ScriptedEngine(max_seq_len=5)
    rs = generate(eng, [[1, 2, 3], [10]], max_tokens=10, temperature=0.0, stop_token_ids=[])
    assert rs[0].finish_reason == "context" and len(rs[0].tokens) == 2      # 3 + 2 = 5 positions
    assert rs[1].finish_reason == "context" and len(rs[1].tokens) == 4
    with pytest.raises(InferenceError, match="exceeds max_seq"):
        generate(eng, [[1] * 6])
    with pytest.raises(InferenceError, match="empty prompt"):
        generate(eng, [[]])


def test_pages_running_out_end_with_context():
    eng = ScriptedEngine(max_batch=2, max_tokens=64 * 2, max_seq_len=1000)
    eng.spec = type("S", (), {"stop_token_ids": [], "bos_token_id": None, "vocab_size": 16})()
    rs = generate(eng, [[1] * 60, [2] * 60], max_tokens=100, temperature=0.0)
    # a request that may come to 160 tokens is planned with all the pages there are (2), so
    # the two run one after the other, and each ends when its second page is full
    assert all(r.finish_reason == "context" for r in rs)
    assert all(len(r.tokens) == 69 for r in rs)      # 68 run to fill the page, the last is emitted only
    eng.cache.check()


def test_plan_batches():
    assert plan_batches([5, 5, 5], 10, 2, 100, 1000) == [[0, 1], [2]]
    pages = lambda n: (n + 63) // 64 * 64
    assert plan_batches([60, 60, 60], 10, 8, 1000, 256, pages) == [[0, 1], [2]]     # 128 tokens each of 256
    assert plan_batches([60, 60, 60], 10, 8, 1000, 256) == [[0, 1, 2]]              # counted as they are: 70 each
    assert plan_batches([], 10, 2, 100, 10) == []


def test_the_loop_asks_the_cache_in_tokens_only():
    """The loop works with any cache that answers token_capacity / tokens_needed / can_grow:
    here one without pages, which counts tokens as they are."""
    class TokenCache:
        def __init__(self, capacity):
            self.capacity, self.lens, self.free = capacity, {}, [1, 0]

        def token_capacity(self):
            return self.capacity

        def tokens_needed(self, n):
            return n

        def can_grow(self, slot, by=1):
            return sum(self.lens.values()) + by <= self.capacity

    eng = ScriptedEngine(max_batch=2, max_seq_len=1000)
    eng.spec = type("S", (), {"stop_token_ids": [], "bos_token_id": None, "vocab_size": 16})()
    cache = TokenCache(50)
    eng.cache = cache
    eng.alloc_slot = lambda: (cache.lens.__setitem__(cache.free[-1], 0), cache.free.pop())[1]
    eng.free_slot = lambda s: (cache.lens.pop(s), cache.free.append(s))
    def step(entries, want):
        for s, t in entries:
            cache.lens[s] += len(t)
        return [(t[-1] + 1) % 16 for _, t in entries]
    eng.step = step
    rs = generate(eng, [[1] * 20, [2] * 20], max_tokens=100, temperature=0.0)
    # each may come to 120 tokens and is planned with all 50: one after the other, each until 50 are held
    assert [r.finish_reason for r in rs] == ["context", "context"]
    assert [len(r.tokens) for r in rs] == [31, 31]
    assert not cache.lens


def test_uniform_is_keyed_by_seed_sequence_and_count():
    a = [uniform(0, 3, n) for n in range(50)]
    assert all(0.0 <= u < 1.0 for u in a) and len(set(a)) == 50
    assert a == [uniform(0, 3, n) for n in range(50)]
    assert uniform(1, 3, 0) != a[0] and uniform(0, 4, 0) != a[0]
    assert abs(sum(uniform(7, i, 0) for i in range(2000)) / 2000 - 0.5) < 0.03


def test_decode_attention_split_rule(monkeypatch):
    """How many workgroups share the pages of one (sequence, kv head) in decode attention:
    none up to 15 pages, two from 16 pages, four from 32 and so on to at most 16, and never more than gives
    every compute unit about one workgroup; a module attribute overrides the rule for tests."""
    from rbitnet_amd.engine import context
    from rbitnet_amd.engine.context import decode_splits, split_bucket
    assert [split_bucket(n) for n in (1, 64, 960, 961, 1024, 2047, 2049, 4096, 8192, 10 ** 6)] == \
        [1, 1, 1, 2, 2, 4, 4, 8, 16, 16]
    assert split_bucket(0) == 1
    # a bucket's contexts reach so many pages and no more (the captured step's page tables are that wide)
    from rbitnet_amd.engine.context import bucket_max_pages
    for b in (1, 2, 4, 8):
        assert split_bucket(64 * bucket_max_pages(b)) == b and split_bucket(64 * bucket_max_pages(b) + 1) == 2 * b
    assert bucket_max_pages(16) is None
    assert decode_splits(8, 8, split_bucket(600), 256) == 1
    assert decode_splits(8, 8, split_bucket(4096), 256) == 4     # 256 // (8 * 8)
    assert decode_splits(1, 8, split_bucket(4096), 256) == 8
    assert decode_splits(64, 8, split_bucket(65536), 256) == 1
    assert decode_splits(1, 1, 16, 256) == 16
    assert decode_splits(8, 8, 16, n_compute_units=128) == 2     # a smaller GPU
    monkeypatch.setattr(context, "FORCED_DECODE_SPLITS", 3)
    assert decode_splits(64, 8, 1, 256) == 3
