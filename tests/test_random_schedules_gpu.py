"""Schedules drawn at random (with a fixed seed): sequences that bring unequal pieces on unequal pasts and pause
in between, through `Engine.step`, each schedule three times with other tokens so that recorded steps are
replayed; and requests of random lengths and limits through `Engine.generate` in batches of random sizes.  Both
against the plain implementation."""
import numpy as np
import pytest
import torch

from functools import lru_cache

from helpers import CONFIGS, TOL, max_err, model_folder
from plain_llama import PlainLlama, argmax_token

pytestmark = pytest.mark.gpu


@lru_cache(maxsize=None)
def _plain(name, rounding=False):
    """The plain implementation in its forms for whole rows (the loops take minutes here)."""
    return PlainLlama.from_folder(model_folder(name), round_bf16=rounding, rows_at_once=True)


def _schedule(rng, totals):
    done, steps = [0] * len(totals), []
    while any(d < t for d, t in zip(done, totals)):
        live = [i for i in range(len(totals)) if done[i] < totals[i]]
        chosen = [i for i in live if rng.random() < 0.7] or [live[0]]
        step = {}
        for i in chosen:
            step[i] = int(min(totals[i] - done[i], rng.choice([1, 1, 1, 2, 5, 17, 40, 64])))
            done[i] += step[i]
        steps.append(step)
    return steps


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_random_step_schedules(name, dtype):
    import rbitnet_amd
    rng = np.random.default_rng(sum(map(ord, name + dtype)))
    cfg = CONFIGS[name][0]
    eng = rbitnet_amd.Engine.load_path(model_folder(name), dtype=dtype, max_batch=5, max_tokens=5 * 192)
    for _ in range(10):
        totals = [int(rng.integers(1, min(cfg["max_position_embeddings"], 150))) for _ in range(int(rng.integers(1, 6)))]
        schedule = _schedule(rng, totals)
        for _ in range(3):
            seqs = [[int(t) for t in rng.integers(0, cfg["vocab_size"], size=n)] for n in totals]
            want = [_plain(name).logits(s) for s in seqs]
            slots = [eng.alloc_slot() for _ in totals]
            at = [0] * len(totals)
            for step in schedule:
                order = list(step)
                logits = eng.step([(slots[i], seqs[i][at[i]:at[i] + step[i]]) for i in order], "all").cpu()
                off = 0
                for i in order:
                    got, span = logits[off:off + step[i]], slice(at[i], at[i] + step[i])
                    off += step[i]
                    err = max_err(got, want[i][span])
                    if err >= TOL[dtype]:      # bfloat16, rarely: no further from exact than rounding alone takes it
                        assert dtype == "bfloat16"
                        rounded = _plain(name, True).logits(seqs[i])[span]
                        assert err < 1.5 * max_err(rounded, want[i][span]), (totals, schedule, i, at[i])
                    at[i] += step[i]
            for s in slots:
                eng.free_slot(s)
            eng.cache.check()
    assert eng.plans.stats["replayed"] > 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_random_requests_through_generate(dtype):
    import rbitnet_amd
    rng = np.random.default_rng(11 if dtype == "float32" else 12)
    for name in ("A", "B", "D"):
        cfg = CONFIGS[name][0]
        for use_graphs in (True, True, False):
            max_batch = int(rng.integers(1, 7))
            eng = rbitnet_amd.Engine.load_path(model_folder(name), dtype=dtype, max_batch=max_batch,
                                               max_tokens=192 * max_batch)
            eng.use_graphs = use_graphs
            n_req = int(rng.integers(2, 16))
            limits = [int(rng.integers(1, 33)) for _ in range(n_req)]
            prompts = [[int(t) for t in rng.integers(0, cfg["vocab_size"], size=int(rng.integers(1, 60)))]
                       for _ in range(n_req)]
            stop = sorted(set(int(t) for t in rng.integers(0, cfg["vocab_size"], size=2)) |
                          set(int(t) for t in eng.spec.stop_token_ids))
            results = eng.generate(prompts, max_tokens=limits, temperature=0.0, stop_token_ids=stop)
            for p, r, limit in zip(prompts, results, limits):
                seq = list(p)
                for tok in r.tokens:               # the engine's own path, every choice judged by the plain logits
                    row = _plain(name).logits(seq, last=1)[-1]
                    best = argmax_token(row)
                    bound = 1e-4 if dtype == "float32" else 0.05 * float(row.abs().max())
                    assert tok == best or float(row[best] - row[tok]) < bound, (name, use_graphs, len(seq))
                    assert tok not in stop
                    seq.append(tok)
                assert (len(r.tokens) == limit) if r.finish_reason == "length" else (len(r.tokens) < limit)
            assert eng.cache.slots.n_held == 0
            eng.cache.check()
