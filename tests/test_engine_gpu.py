"""The engine against the plain implementation, in float32 and bfloat16: whole requests,
the last 32 tokens one by one, and batches of unequal lengths with slot reuse."""
import pytest
import torch

from helpers import TOL, max_err, model_folder, plain_logits, tokens_for

pytestmark = pytest.mark.gpu

LENGTHS = {"A": [5, 17, 32, 70], "B": [1, 9, 40, 77], "C": [3, 64, 65, 150]}


def _engine(name, dtype, **kw):
    import rbitnet_amd
    return rbitnet_amd.Engine.load_path(model_folder(name), dtype=dtype, max_tokens=kw.pop("max_tokens", 1024), **kw)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_whole_requests(name, dtype):
    eng = _engine(name, dtype)
    for i, n in enumerate(LENGTHS[name]):
        toks = tokens_for(name, n, i)
        slot = eng.alloc_slot()
        got = eng.step([(slot, toks)], "all")
        eng.free_slot(slot)
        err = max_err(got, plain_logits(name, tuple(toks)))
        assert err < TOL[dtype], f"{name} {dtype} length {n}: {err}"
    eng.cache.check()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_last_32_one_by_one(name, dtype):
    eng = _engine(name, dtype)
    for i, n in enumerate(LENGTHS[name]):
        toks = tokens_for(name, n, i)
        want = plain_logits(name, tuple(toks))
        head = max(0, n - 32)
        slot = eng.alloc_slot()
        rows = []
        if head:
            rows.append(eng.step([(slot, toks[:head])], "all"))
        for t in toks[head:]:
            rows.append(eng.step([(slot, [t])], "last"))
        eng.free_slot(slot)
        got = torch.cat(rows)
        err = max_err(got, want)
        assert err < TOL[dtype], f"{name} {dtype} length {n}: {err}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_unequal_batches_with_slot_reuse(name, dtype):
    """Two batches one after the other in an engine with just enough slots: prompts of
    unequal lengths in one step, then one token each; shorter requests end earlier."""
    lengths = LENGTHS[name]
    eng = _engine(name, dtype, max_batch=len(lengths), max_tokens=64 * sum((n + 63) // 64 for n in lengths))
    for round_ in range(2):
        # what earlier sequences left in the pages must not matter: poison all of it
        for g in eng.cache.kv_groups:
            g.k.fill_(float("nan"))
            g.v.fill_(float("nan"))
        reqs = [tokens_for(name, n, 10 * round_ + i) for i, n in enumerate(lengths)]
        prompt_len = [max(1, len(r) - (3 + 5 * i)) for i, r in enumerate(reqs)]
        slots = [eng.alloc_slot() for _ in reqs]
        got = [[] for _ in reqs]
        logits = eng.step([(s, r[:p]) for s, r, p in zip(slots, reqs, prompt_len)], "all")
        off = 0
        for i, p in enumerate(prompt_len):
            got[i].append(logits[off:off + p])
            off += p
        done = list(prompt_len)
        live = [i for i in range(len(reqs)) if done[i] < len(reqs[i])]
        for i in range(len(reqs)):
            if i not in live:
                eng.free_slot(slots[i])
        while live:
            logits = eng.step([(slots[i], [reqs[i][done[i]]]) for i in live], "last")
            for j, i in enumerate(live):
                got[i].append(logits[j:j + 1])
                done[i] += 1
            for i in [i for i in live if done[i] >= len(reqs[i])]:
                eng.free_slot(slots[i])
            live = [i for i in live if done[i] < len(reqs[i])]
        eng.cache.check()
        assert eng.cache.slots.n_held == 0
        for i, r in enumerate(reqs):
            err = max_err(torch.cat(got[i]), plain_logits(name, tuple(r)))
            assert err < TOL[dtype], f"{name} {dtype} round {round_} request {i}: {err}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C"])
def test_batch_that_shrinks_from_20_sequences_to_8(name, dtype):
    """Steps of more than 16 tokens and of at most 16 run different kernels (with few tokens the
    products do the residual sums and the norms themselves).  20 sequences decode together,
    12 of them end after two tokens and the other 8 go on: every sequence's logits match the
    plain implementation on both sides of the change."""
    n = 20
    reqs = [tokens_for(name, 4 + i + (2 if i % 5 < 3 else 6), 40 + i) for i in range(n)]
    prompt_len = [4 + i for i in range(n)]
    eng = _engine(name, dtype, max_batch=n, max_tokens=64 * n)
    slots = [eng.alloc_slot() for _ in reqs]
    got = [[] for _ in reqs]
    logits = eng.step([(s, r[:p]) for s, r, p in zip(slots, reqs, prompt_len)], "last")
    for i in range(n):
        got[i].append(logits[i:i + 1])
    done = list(prompt_len)
    live = list(range(n))
    sizes = []
    while live:
        sizes.append(len(live))
        logits = eng.step([(slots[i], [reqs[i][done[i]]]) for i in live], "last")
        for j, i in enumerate(live):
            got[i].append(logits[j:j + 1])
            done[i] += 1
        for i in [i for i in live if done[i] >= len(reqs[i])]:
            eng.free_slot(slots[i])
        live = [i for i in live if done[i] < len(reqs[i])]
    assert sizes == [20, 20, 8, 8, 8, 8]
    eng.cache.check()
    for i, r in enumerate(reqs):
        want = plain_logits(name, tuple(r))[prompt_len[i] - 1:]
        err = max_err(torch.cat(got[i]), want)
        assert err < TOL[dtype], f"{name} {dtype} request {i}: {err}"
