"""Generation through the Python entry point and the command line, long decoding, the
first tokens of a sequence, sampling that does not depend on the batch."""
import json
import os
import subprocess
import sys

import pytest
import torch

from helpers import TOL, max_err, model_folder, plain_logits, tokens_for
from plain_llama import argmax_token, sample_token

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _engine(name, dtype, **kw):
    import rbitnet_amd
    kw.setdefault("max_tokens", 2048)
    return rbitnet_amd.Engine.load_path(model_folder(name), dtype=dtype, **kw)


def _plain_greedy(name, prompt, n, stop=()):
    """Greedy continuation by the plain implementation, with the margin between the best
    and the second logit at each step (a tiny margin means either token is right)."""
    seq, out, margins = list(prompt), [], []
    for _ in range(n):
        row = plain_logits(name, tuple(seq))[-1]
        top = torch.topk(row, 2).values
        tok = argmax_token(row)
        if tok in stop:
            break
        margins.append(float(top[0] - top[1]))
        out.append(tok)
        seq.append(tok)
    return out, margins


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_matches_plain_float32(name):
    eng = _engine(name, "float32", max_batch=3)
    prompts = [tokens_for(name, n, 40 + i) for i, n in enumerate([5, 17, 32, 1])]
    results = eng.generate(prompts, max_tokens=16, temperature=0.0, stop_token_ids=[])
    for p, r in zip(prompts, results):
        want, margins = _plain_greedy(name, p, 16)
        assert min(margins) > 1e-4, "test data: a near tie, pick another seed"
        assert r.tokens == want and r.finish_reason == "length"
    # the same call twice gives the same tokens (the reference's determinism test, toy.rs:121-127)
    again = eng.generate(prompts, max_tokens=16, temperature=0.0, stop_token_ids=[])
    assert [r.tokens for r in again] == [r.tokens for r in results]
    assert eng.cache.slots.n_held == 0
    eng.cache.check()


def test_stop_token_ends_generation_and_is_not_emitted():
    eng = _engine("A", "float32")
    prompt = tokens_for("A", 9, 3)
    want, _ = _plain_greedy("A", prompt, 12)
    stop = want[4]
    first = want.index(stop)
    (r,) = eng.generate([prompt], max_tokens=12, temperature=0.0, stop_token_ids=[stop])
    assert r.tokens == want[:first] and r.finish_reason == "stop"


def test_bfloat16_greedy_agrees_where_the_margin_is_clear():
    eng = _engine("C", "bfloat16")
    prompt = tokens_for("C", 20, 5)
    (r,) = eng.generate([prompt], max_tokens=24, temperature=0.0, stop_token_ids=[])
    seq = list(prompt)
    for tok in r.tokens:                       # follow the engine's own path and judge each choice
        row = plain_logits("C", tuple(seq))[-1]
        best = argmax_token(row)
        if tok != best:
            assert float(row[best] - row[tok]) < 0.05 * float(row.abs().max()), "a clear best token was missed"
        seq.append(tok)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(dtype):
    """A short prompt and then 300 tokens one by one across several pages: every logit row
    against the plain implementation run on the whole sequence."""
    name = "C"
    toks = tokens_for(name, 310, 77)
    want = plain_logits(name, tuple(toks))
    eng = _engine(name, dtype)
    slot = eng.alloc_slot()
    rows = [eng.step([(slot, toks[:10])], "all")]
    for t in toks[10:]:
        rows.append(eng.step([(slot, [t])], "last"))
    eng.free_slot(slot)
    got = torch.cat(rows).cpu().double()
    err = (got - want).abs().amax(dim=1) / want.abs().max()
    assert float(err.max()) < TOL[dtype], f"worst position {int(err.argmax())}: {float(err.max())}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decoding_where_the_split_count_changes(dtype):
    """Decode attention deals a sequence's pages to more workgroups as the context grows (one
    split up to 15 pages, two from 16 pages on), and the captured step is kept per split
    count.  Logits from 940 to 990 keys against the plain implementation, replayed as
    graphs and launched one by one."""
    name = "D"
    toks = tokens_for(name, 990, 5)
    want = plain_logits(name, tuple(toks))
    for graphs in (True, False):
        eng = _engine(name, dtype, max_tokens=1088, max_batch=1)
        assert eng.use_graphs
        eng.use_graphs = graphs
        slot = eng.alloc_slot()
        assert eng.step([(slot, toks[:940])], [[]]).shape[0] == 0
        rows = []
        for t in toks[940:]:
            eng.decode_step([slot], [t])
            rows.append(eng.last_decode_logits.float().cpu().clone())
        if graphs:
            assert sorted(b for _, b in eng._graphs) == [1, 2]
        eng.free_slot(slot)
        got = torch.cat(rows).double()
        err = (got - want[940:]).abs().amax(dim=1) / want.abs().max()
        assert float(err.max()) < TOL[dtype], f"graphs={graphs}: worst position {940 + int(err.argmax())}: {float(err.max())}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_first_tokens_of_a_sequence(name, dtype):
    """Positions 0, 1, 2 alone and together: a one-token sequence attends to itself only."""
    toks = tokens_for(name, 3, 9)
    want = plain_logits(name, tuple(toks))
    eng = _engine(name, dtype)
    for cut in ([3], [1, 2], [1, 1, 1], [2, 1]):
        slot = eng.alloc_slot()
        rows, at = [], 0
        for n in cut:
            rows.append(eng.step([(slot, toks[at:at + n])], "all"))
            at += n
        eng.free_slot(slot)
        assert max_err(torch.cat(rows), want) < TOL[dtype], cut


def test_temperature_sampling_does_not_depend_on_the_batch():
    eng = _engine("B", "float32", max_batch=4)
    prompts = [tokens_for("B", n, 60 + i) for i, n in enumerate([1, 9, 40, 77])]
    together = eng.generate(prompts, max_tokens=24, temperature=0.8, seed=5, stop_token_ids=[])
    eng1 = _engine("B", "float32", max_batch=1)
    alone = eng1.generate(prompts, max_tokens=24, temperature=0.8, seed=5, stop_token_ids=[])
    assert [r.tokens for r in together] == [r.tokens for r in alone]
    other = eng.generate(prompts, max_tokens=24, temperature=0.8, seed=6, stop_token_ids=[])
    assert [r.tokens for r in other] != [r.tokens for r in together]
    # the first sampled token of each request against the plain inverse CDF
    from rbitnet_amd.sampling import uniform
    for i, (p, r) in enumerate(zip(prompts, together)):
        row = plain_logits("B", tuple(p))[-1]
        assert r.tokens[0] == sample_token(row, 0.8, uniform(5, i, 0))


def test_step_refuses_what_it_cannot_run():
    from rbitnet_amd.errors import CacheError, InferenceError
    eng = _engine("A", "float32", max_tokens=128, max_batch=2)
    s = eng.alloc_slot()
    with pytest.raises(InferenceError, match="token id out of range"):
        eng.step([(s, [256])])
    with pytest.raises(InferenceError, match="position >= max_seq"):
        eng.step([(s, [1] * 129)])
    with pytest.raises(InferenceError, match="at least one token"):
        eng.step([(s, [])])
    with pytest.raises(InferenceError, match="wanted place"):
        eng.step([(s, [1, 2])], [[2]])
    assert eng.length(s) == 0
    s2 = eng.alloc_slot()
    eng.step([(s, [1] * 70)])
    with pytest.raises(CacheError, match="cache full"):
        eng.step([(s2, [1])])                  # both pages are held by the first sequence
    with pytest.raises(CacheError):
        eng.alloc_slot()
    eng.free_slot(s)
    eng.step([(s2, [1])])


def test_command_line_generate_and_inspect(tmp_path):
    env = dict(os.environ, PYTHONPATH=ROOT)
    folder = model_folder("A")
    prompt = tokens_for("A", 7, 21)
    want, _ = _plain_greedy("A", prompt, 5)
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "rbitnet"), "generate", "--model", folder,
                          "--dtype", "float32", "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "5",
                          "--temperature", "0"], capture_output=True, text=True, env=env, timeout=300)
    assert out.returncode == 0, out.stderr
    rec = json.loads(out.stdout.strip().splitlines()[-1])
    assert rec["tokens"] == want and rec["finish_reason"] == "length" and rec["prompt_tokens"] == 7
    bad = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "rbitnet"), "generate", "--model",
                          str(tmp_path / "none"), "--prompt-ids", "1"], capture_output=True, text=True, env=env)
    assert bad.returncode == 1 and bad.stderr.startswith("error: ")
    ins = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "rbitnet"), "inspect", folder],
                         capture_output=True, text=True, env=env)
    assert ins.returncode == 0 and "tensors=21" in ins.stdout and "... and 1 more" in ins.stdout


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_graph_decode_equals_launch_by_launch(dtype):
    """The captured decode step against the same kernels launched one by one: the same
    tokens and logits on every replay, with eager work and synchronisations in between,
    across a page boundary, and for a batch that shrinks."""
    name = "C"
    eng_g = _engine(name, dtype, max_batch=3)
    eng_e = _engine(name, dtype, max_batch=3)
    eng_e.use_graphs = False
    assert eng_g.use_graphs
    prompts = [tokens_for(name, n, 30 + i) for i, n in enumerate([60, 5, 130])]
    outs = []
    for eng in (eng_g, eng_e):
        slots = [eng.alloc_slot() for _ in prompts]
        logits = eng.step(list(zip(slots, prompts)), "last")
        toks = eng.sampler.sample(logits)
        hist = [list(toks)]
        for step in range(12):
            if step == 8:                       # the shortest request leaves
                eng.free_slot(slots.pop(1))
                toks.pop(1)
            temps = [0.0, 0.9, 0.0][:len(slots)]
            us = [0.1 * (step % 7), 0.37, 0.5][:len(slots)]
            toks = eng.decode_step(slots, toks, temps, us)
            hist.append(list(toks))
            if eng.use_graphs:
                g = next(gr for (n, _), gr in eng._graphs.items() if n == len(slots))
                hist.append(g.logits.float().cpu().clone())
                torch.cuda.synchronize()
                _ = (torch.ones(1000, device="cuda") * 2).sum().item()      # unrelated eager work
            else:
                hist.append(None)
        outs.append(hist)
        for s in slots:
            eng.free_slot(s)
        eng.cache.check()
    tok_g = [h for h in outs[0] if isinstance(h, list)]
    tok_e = [h for h in outs[1] if isinstance(h, list)]
    assert tok_g == tok_e
    # and the graph's logits against the plain implementation at the last step
    seq0 = prompts[0] + [t[0] for t in tok_g[:-1]]
    last = [h for h in outs[0] if isinstance(h, torch.Tensor)][-1]
    assert max_err(last[0:1], plain_logits(name, tuple(seq0))[-1:]) < TOL[dtype]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C"])
def test_idle_rows_of_a_captured_step_touch_no_live_sequence(name, dtype):
    """Captured steps exist for a ladder of sizes; a batch of 5 runs in 6 rows, then, as sequences
    leave one by one, in 4, 3, 2 and 1.  Between two steps the cache may change at the live
    sequences' new positions and in the spare page and nowhere else; every live row's logits
    match the plain implementation; the state of the free lists stays sound."""
    from rbitnet_amd.engine.decode_graph import graph_size
    assert [graph_size(n) for n in (1, 2, 3, 4, 5, 6, 7, 9, 13, 17, 20, 33, 49, 64, 65, 97, 200)] == \
        [1, 2, 3, 4, 6, 6, 8, 12, 16, 24, 24, 48, 64, 64, 96, 128, 224]
    lengths = [70, 5, 64, 33, 12]
    reqs = [tokens_for(name, n + 9, 80 + i) for i, n in enumerate(lengths)]
    eng = _engine(name, dtype, max_batch=5, max_tokens=64 * 8)
    assert eng.use_graphs
    groups = eng.cache.kv_groups
    for g in groups:
        g.k.fill_(3.0)
        g.v.fill_(3.0)
    slots = [eng.alloc_slot() for _ in reqs]
    eng.step([(s, r[:n]) for s, r, n in zip(slots, reqs, lengths)], [[] for _ in reqs])
    live = list(range(len(reqs)))
    sizes = []
    for j in range(9):
        before = [(g.k.clone(), g.v.clone()) for g in groups]
        lens = [eng.cache.length(slots[i]) for i in live]
        eng.cache.reserve([slots[i] for i in live], [1] * len(live))      # so that the pages of this step are known here
        tables = eng.cache.block_tables([slots[i] for i in live])
        eng.decode_step([slots[i] for i in live], [reqs[i][lengths[i] + j] for i in live])
        sizes.append(graph_size(len(live)))
        got = eng.last_decode_logits.float().cpu()
        assert got.shape[0] == len(live)
        for row, i in enumerate(live):
            want = plain_logits(name, tuple(reqs[i]))[lengths[i] + j]
            assert max_err(got[row:row + 1], want[None]) < TOL[dtype], (j, i)
        for g, (k0, v0) in zip(groups, before):
            allowed = torch.zeros(g.k.shape[1], 64, dtype=torch.bool, device=g.k.device)
            allowed[g.spare_page] = True
            for pages, n in zip(tables[id(g)], lens):
                allowed[pages[n // 64], n % 64] = True
            for new, old in ((g.k, k0), (g.v, v0)):
                changed = (new != old).any(dim=4).any(dim=2).any(dim=0)        # [pages, 64]
                assert not bool((changed & ~allowed).any()), f"step {j}: a position outside the step's own was written"
        if j in (1, 3, 5, 6):                                       # a sequence leaves: 5, 4, 3, 2, 1
            eng.free_slot(slots[live.pop(1 if len(live) > 1 else 0)])
    assert sizes == [6, 6, 4, 4, 3, 3, 2, 1, 1]
    assert sorted(n for n, _ in eng._graphs) == [1, 2, 3, 4, 6]
    for i in live:
        eng.free_slot(slots[i])
    eng.cache.check()
    assert eng.cache.slots.n_held == 0
