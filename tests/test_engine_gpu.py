"""The engine against the plain implementation, in float32 and bfloat16: whole requests,
the last 32 tokens one by one, and batches of unequal lengths with slot reuse."""
import pytest
import torch

from helpers import (BF16_MAX_RATIO, BF16_RMS_RATIO, BF16_RMS_RATIO_FEW, CONFIGS, TOL, max_err, model_folder,
                     plain_logits, plain_logits_rounded, rms_err, tokens_for)

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
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_prompts_in_pieces_for_several_sequences_at_once(name, dtype):
    """Steps that bring several tokens per sequence on top of pasts that differ per sequence (a
    prompt fed in pieces, batched): pieces that end inside a page, at its edge and beyond it, a
    sequence that brings one token while its neighbours bring many."""
    lengths = [125, 64, 75]
    cuts = [[60, 5, 64], [4, 59, 1], [61, 0, 10]]           # tokens per sequence and step; 0: it sits the step out
    reqs = [tokens_for(name, n, 60 + i) for i, n in enumerate(lengths)]
    eng = _engine(name, dtype, max_batch=3, max_tokens=64 * 5)
    for g in eng.cache.kv_groups:
        g.k.fill_(float("nan"))
        g.v.fill_(float("nan"))
    slots = [eng.alloc_slot() for _ in reqs]
    done = [0] * len(reqs)
    got = [[] for _ in reqs]
    for cut in cuts:
        live = [i for i, n in enumerate(cut) if n]
        logits = eng.step([(slots[i], reqs[i][done[i]:done[i] + cut[i]]) for i in live], "all")
        off = 0
        for i in live:
            got[i].append(logits[off:off + cut[i]])
            off += cut[i]
            done[i] += cut[i]
    assert done == lengths
    for i, r in enumerate(reqs):
        err = max_err(torch.cat(got[i]), plain_logits(name, tuple(r)))
        assert err < TOL[dtype], f"{name} {dtype} request {i}: {err}"


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


@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_bfloat16_error_is_the_cost_of_rounding_and_no_more(name):
    """The bound of 3e-2 on the bfloat16 engine is loose enough to let a systematic error of a
    per cent pass.  What rounding to bfloat16 must cost is measured here by the plain
    implementation rounding at the places where the engine stores bfloat16; the engine's error
    against the exact logits may be that large and little more, as a root mean square over each
    request's logits and at its worst logit.  Steps of at most 16 tokens fold the norms into the
    products around them and round bf16(x * gain) instead of bf16(x * gain / rms): the same cost."""
    cap = CONFIGS[name][0]["max_position_embeddings"]
    eng = _engine(name, "bfloat16", max_tokens=1152)
    for i, n in enumerate([40, 77, 150, 700]):
        if n > cap:
            continue
        toks = tokens_for(name, n, 20 + i)
        exact = plain_logits(name, tuple(toks))
        rounded = plain_logits_rounded(name, tuple(toks))
        slot = eng.alloc_slot()
        got = eng.step([(slot, toks[:n - 8])], "all")
        tail = torch.cat([eng.step([(slot, [t])], "last") for t in toks[n - 8:]])
        eng.free_slot(slot)
        head, last = slice(0, n - 8), slice(n - 8, n)
        cost = rms_err(rounded[head], exact[head])
        assert 1e-4 < cost < 1e-2                               # the plain implementation does round
        assert rms_err(got, exact[head]) < BF16_RMS_RATIO * cost, f"{name} length {n}"
        assert max_err(got, exact[head]) < BF16_MAX_RATIO * max_err(rounded[head], exact[head]), f"{name} length {n}"
        assert rms_err(tail, exact[last]) < BF16_RMS_RATIO_FEW * rms_err(rounded[last], exact[last]), f"{name} length {n}"


def test_folder_with_adjacent_pairs_and_permuted_rows_gives_the_same_logits(tmp_path):
    """A weight file whose q and k rows were permuted for the reference's pairing of the rotation
    (model.rs:122-136), read with "interleaved", against the same model un-permuted, read with
    "half": the engine's two pairings are the same function."""
    import json
    import rbitnet_amd
    from safetensors.torch import load_file, save_file
    cfg = dict(CONFIGS["B"][0])
    assert "rope_style" not in cfg
    src = model_folder("B")
    d = cfg["hidden_size"] // cfg["num_attention_heads"]
    perm = torch.stack([torch.arange(d // 2), torch.arange(d // 2) + d // 2], dim=1).reshape(-1)
    tensors = load_file(f"{src}/model.safetensors")
    for key in list(tensors):
        if key.endswith("q_proj.weight") or key.endswith("k_proj.weight"):
            w = tensors[key]
            tensors[key] = w.view(-1, d, w.shape[1])[:, perm, :].reshape(w.shape).contiguous()
    dst = tmp_path / "permuted"
    dst.mkdir()
    save_file(tensors, str(dst / "model.safetensors"))
    with open(dst / "config.json", "w") as f:
        json.dump(dict(cfg, rope_style="interleaved"), f)
    toks = tokens_for("B", 50, 3)
    want = plain_logits("B", tuple(toks))
    for folder in (src, str(dst)):
        eng = rbitnet_amd.Engine.load_path(folder, dtype="float32", max_tokens=128)
        slot = eng.alloc_slot()
        assert max_err(eng.step([(slot, toks)], "all"), want) < TOL["float32"]
        eng.free_slot(slot)


def test_cache_for_a_configuration_with_a_very_long_context(tmp_path, monkeypatch, capfd):
    """config.json files of real checkpoints allow 131,072 positions.  Without sizes from the caller
    the cache is made for 8 such sequences if that fits the free memory, and for what fits
    otherwise (with a message); a request beyond what fits ends with "context"; a size asked for
    that does not fit is an error that says what would."""
    import rbitnet_amd
    from rbitnet_amd.errors import CacheError
    cfg = dict(CONFIGS["A"][0], max_position_embeddings=131072)
    folder = rbitnet_amd.write_random_model(str(tmp_path / "m"), cfg, seed=0, std=0.1)
    per_token = 2 * cfg["num_hidden_layers"] * cfg["num_key_value_heads"] * 16 * 2        # k and v, bfloat16
    eng = rbitnet_amd.Engine.load_path(folder)
    assert eng.max_seq_len == 131072 and eng.cache.bytes() == (8 * 131072 + 64) * per_token      # and the spare page
    eng_aside = eng.model.activation_bytes(8192)
    assert eng_aside > 1 << 20
    del eng
    real = torch.cuda.mem_get_info
    # what a cache nobody sized leaves alone: room for the activations of a long step; beyond that, 1 MiB is free
    aside = eng_aside
    monkeypatch.setattr(torch.cuda, "mem_get_info", lambda *a: (aside + (1 << 20), real(*a)[1]))
    eng = rbitnet_amd.Engine.load_path(folder)
    fits = int((1 << 20) * 0.9) // per_token // 64 * 64
    assert eng.cache.bytes() == (fits + 64) * per_token and eng.cache.token_capacity() == fits
    assert "sized to the" in capfd.readouterr().err
    (r,) = eng.generate([tokens_for("A", fits - 10, 1)], max_tokens=100, temperature=0.0, stop_token_ids=[])
    assert r.finish_reason == "context" and len(r.tokens) == 11       # ten run, the last is only emitted
    eng.cache.check()
    with pytest.raises(CacheError, match="does not fit"):
        rbitnet_amd.Engine.load_path(folder, max_tokens=1 << 20)
    # the position limit of the reference (model.rs:221-223) still holds
    small = rbitnet_amd.Engine.load_path(folder, max_seq_len=100, max_tokens=256)
    slot = small.alloc_slot()
    from rbitnet_amd.errors import InferenceError
    with pytest.raises(InferenceError, match="max_seq"):
        small.step([(slot, tokens_for("A", 101, 2))], "last")
