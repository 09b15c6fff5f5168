"""The kernels that only wide models select (256 x 256 tiles, the token-resident and the
panel products, flash attention over many blocks, decode splits) at the widths of Llama-3-8B
and Llama-2-7B with two layers and of Llama-3.1-70B with one: the float32 and the bfloat16
engine against the plain implementation, for batches of unequal lengths whose longest request
spans five pages of the cache, the last tokens one by one, one batch after another in the same
slots; the captured decode step (`Engine.decode_step`, the path that generation and the
benchmark run) alone and with twenty sequences while the longest context crosses the length at
which decode attention is split; prompts that arrive in pieces for several sequences at once.
Then the bfloat16 engine's drift from the float32 engine over twenty requests."""
import os
import sys

import numpy as np
import pytest
import torch

sys.path.insert(0, os.path.dirname(__file__))

pytestmark = pytest.mark.gpu

WIDE = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 4096, "num_hidden_layers": 2,
    "num_attention_heads": 32, "num_key_value_heads": 8, "intermediate_size": 14336, "vocab_size": 128256,
    "rope_theta": 500000.0, "rms_norm_eps": 1e-5, "max_position_embeddings": 8192,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 1024},
}
WIDER = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 8192, "num_hidden_layers": 1,
    "num_attention_heads": 64, "num_key_value_heads": 8, "intermediate_size": 28672, "vocab_size": 128256,
    "rope_theta": 500000.0, "rms_norm_eps": 1e-5, "max_position_embeddings": 8192,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 8192},
}
# one kv head per head (`n_rep = 1`, model.rs:234,263): the vector decode kernel at head size 128,
# a feed-forward width of 172 K tiles, a vocabulary that is no multiple of 256
MHA = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 4096, "num_hidden_layers": 2,
    "num_attention_heads": 32, "num_key_value_heads": 32, "intermediate_size": 11008, "vocab_size": 32000,
    "rope_theta": 10000.0, "rms_norm_eps": 1e-5, "max_position_embeddings": 4096,
}
CONFIGS = {"wide": WIDE, "wider": WIDER, "mha": MHA}
TAIL = 3                                   # tokens of each request that are fed one by one
BATCHES = {"wide": [[300, 130, 65, 1], [66, 20]], "wider": [[200, 70, 1]], "mha": [[300, 130, 65, 1], [66, 20]]}
# the captured decode step: GRAPH_TAIL tokens of every request are decoded through it.  The first
# request alone, then all twenty together; its context passes 960 keys (15 pages) on the way,
# where the split bucket of decode attention and with it the captured graph change.
GRAPH_TAIL = 6
GRAPH_LENGTHS = {"wide": [963, 130, 65, 300, 7, 31, 64, 200, 90, 17, 450, 33, 257, 129, 8, 512, 77, 256, 40, 100],
                 "wider": [963, 70, 9, 130, 64, 33, 200, 17, 65, 100, 7, 257, 40, 90, 31, 129, 77, 8, 12, 300],
                 "mha": [963, 130, 65, 300, 7, 31, 64, 200, 90, 17, 450, 33, 257, 129, 8, 512, 77, 256, 40, 100]}
# prompts that come in pieces: per request its total length and the sizes of its first pieces
PIECES = {"lengths": [260, 150, 90], "cuts": [[200, 70, 50], [59, 17, 30]]}


def _tokens(kind, lengths, seed):
    rng = np.random.default_rng(seed)
    vocab = CONFIGS[kind]["vocab_size"]
    return [[int(t) for t in rng.integers(0, vocab, size=n)] for n in lengths]


def _requests(kind):
    rng = np.random.default_rng(11)
    vocab = CONFIGS[kind]["vocab_size"]
    return [[[int(t) for t in rng.integers(0, vocab, size=n)] for n in lengths] for lengths in BATCHES[kind]]


@pytest.fixture(scope="module")
def folder(tmp_path_factory):
    import rbitnet_amd
    path = str(tmp_path_factory.mktemp("wide") / "m")
    # std 0.03: large enough for attention and the gate to matter at this width
    return rbitnet_amd.write_random_model(path, WIDE, seed=5, std=0.03, norm_std=0.05, dtype=torch.bfloat16)


@pytest.fixture(scope="module")
def wider_folder(tmp_path_factory):
    import rbitnet_amd
    path = str(tmp_path_factory.mktemp("wider") / "m")
    return rbitnet_amd.write_random_model(path, WIDER, seed=6, std=0.02, norm_std=0.05, dtype=torch.bfloat16)


@pytest.fixture(scope="module")
def mha_folder(tmp_path_factory):
    import rbitnet_amd
    path = str(tmp_path_factory.mktemp("mha") / "m")
    return rbitnet_amd.write_random_model(path, MHA, seed=7, std=0.03, norm_std=0.05, dtype=torch.bfloat16)


def _plain_logits(path, kind):
    """float64 logits of the plain implementation (its sums run on the GPU for their size, in the
    forms for long sequences), computed once per folder: for every request of the batches, for the
    last GRAPH_TAIL positions of the requests of the captured decode step, and for the requests
    that come in pieces."""
    from plain_llama import PlainLlama
    plain = PlainLlama.from_folder(path, device="cuda:0", rows_at_once=True)
    out = {"batches": [[plain.logits(r).cpu() for r in batch] for batch in _requests(kind)],
           "graph": [plain.logits(r, last=GRAPH_TAIL).cpu() for r in _tokens(kind, GRAPH_LENGTHS[kind], 21)],
           "pieces": [plain.logits(r).cpu() for r in _tokens(kind, PIECES["lengths"], 31)]}
    del plain
    torch.cuda.empty_cache()
    return out


@pytest.fixture(scope="module")
def wide_plain(folder):
    return _plain_logits(folder, "wide")


@pytest.fixture(scope="module")
def wider_plain(wider_folder):
    return _plain_logits(wider_folder, "wider")


@pytest.fixture(scope="module")
def mha_plain(mha_folder):
    return _plain_logits(mha_folder, "mha")


def _rel(a, b):
    return float((a.double() - b.double()).abs().max() / b.double().abs().max())


def _batches_against_plain(path, kind, want, dtype, tol):
    """Each batch: the prompts (all but the last TAIL tokens) in one step, then one token each,
    requests with fewer tokens ending earlier; the next batch in the same slots, whose pages are
    filled with NaN in between."""
    import rbitnet_amd
    batches, want = _requests(kind), want["batches"]
    n_slots = max(len(b) for b in batches)
    need = max(sum((len(r) + 63) // 64 * 64 for r in b) for b in batches)
    eng = rbitnet_amd.Engine.load_path(path, dtype=dtype, max_tokens=need, max_batch=n_slots)
    for reqs, logits_want in zip(batches, want):
        for g in eng.cache.kv_groups:
            g.k.fill_(float("nan"))
            g.v.fill_(float("nan"))
        slots = [eng.alloc_slot() for _ in reqs]
        heads = [max(1, len(r) - TAIL) for r in reqs]
        got = [[] for _ in reqs]
        logits = eng.step([(s, r[:h]) for s, r, h in zip(slots, reqs, heads)], "all")
        off = 0
        for i, h in enumerate(heads):
            got[i].append(logits[off:off + h].cpu())
            off += h
        for j in range(TAIL):
            live = [i for i, (r, h) in enumerate(zip(reqs, heads)) if h + j < len(r)]
            if not live:
                break
            logits = eng.step([(slots[i], [reqs[i][heads[i] + j]]) for i in live], "last").cpu()
            for row, i in enumerate(live):
                got[i].append(logits[row:row + 1])
        for s in slots:
            eng.free_slot(s)
        for i, (r, w) in enumerate(zip(reqs, logits_want)):
            g = torch.cat(got[i])
            assert g.shape == w.shape
            err = (g.double() - w).abs().amax(dim=1) / w.abs().max()
            assert float(err.max()) < tol, f"{kind} {dtype}: request of {len(r)} tokens, position {int(err.argmax())}: {float(err.max())}"
    eng.cache.check()
    assert eng.cache.slots.n_held == 0
    del eng
    torch.cuda.empty_cache()


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 3e-2)])
def test_wide_model_against_plain(folder, wide_plain, dtype, tol):
    """Sums over 4,096 and 14,336 terms, a vocabulary of 128,256, 32 heads on 8."""
    _batches_against_plain(folder, "wide", wide_plain, dtype, tol)


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 3e-2)])
def test_wider_model_against_plain(wider_folder, wider_plain, dtype, tol):
    """The widths of the 70B shape: sums over 8,192 and 28,672 terms, 64 heads on 8, the llama3
    rule with its original length of 8,192."""
    _batches_against_plain(wider_folder, "wider", wider_plain, dtype, tol)


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 3e-2)])
def test_mha_model_against_plain(mha_folder, mha_plain, dtype, tol):
    """The widths of the Llama-2-7B shape: a kv head per head, sums over 11,008 terms (172 tiles of
    64, cut into slices that are no power of two), a vocabulary of 32,000."""
    _batches_against_plain(mha_folder, "mha", mha_plain, dtype, tol)


def _captured_decode_against_plain(path, kind, want, dtype, tol):
    """`Engine.decode_step` with graphs on: the first request alone, then all twenty together.
    Every step's logits (`last_decode_logits`) against the plain implementation; the first
    request's context goes from 958 to 963 keys, so both runs change the split bucket on the way
    and replay a second captured graph."""
    import rbitnet_amd
    from rbitnet_amd.engine.decode_graph import graph_size
    reqs, want = _tokens(kind, GRAPH_LENGTHS[kind], 21), want["graph"]
    need = sum((len(r) + 63) // 64 * 64 for r in reqs)
    eng = rbitnet_amd.Engine.load_path(path, dtype=dtype, max_tokens=need, max_batch=len(reqs))
    assert eng.use_graphs
    for chosen in ([0], list(range(len(reqs)))):
        for g in eng.cache.kv_groups:
            g.k.fill_(float("nan"))
            g.v.fill_(float("nan"))
        slots = [eng.alloc_slot() for _ in chosen]
        heads = [len(reqs[i]) - GRAPH_TAIL for i in chosen]
        assert eng.step([(s, reqs[i][:h]) for s, i, h in zip(slots, chosen, heads)], [[] for _ in chosen]).shape[0] == 0
        before = len(eng._graphs)
        for j in range(GRAPH_TAIL):
            eng.decode_step(slots, [reqs[i][h + j] for i, h in zip(chosen, heads)])
            got = eng.last_decode_logits.cpu().double()
            for row, i in enumerate(chosen):
                w = want[i][j]
                err = float((got[row] - w).abs().max() / want[i].abs().max())
                assert err < tol, f"{kind} {dtype}: {len(chosen)} sequences, request {i}, token {j} of its tail: {err}"
        assert sorted(b for n, b in eng._graphs if n == graph_size(len(chosen))) == [1, 2]      # 20 run in 24 rows
        assert len(eng._graphs) == before + 2
        for s in slots:
            eng.free_slot(s)
    eng.cache.check()
    assert eng.cache.slots.n_held == 0
    del eng
    torch.cuda.empty_cache()


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 3e-2)])
def test_wide_model_captured_decode_step_against_plain(folder, wide_plain, dtype, tol):
    """What the benchmark times: the captured decode step at the widths of the 8B shape."""
    _captured_decode_against_plain(folder, "wide", wide_plain, dtype, tol)


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 3e-2)])
def test_wider_model_captured_decode_step_against_plain(wider_folder, wider_plain, dtype, tol):
    _captured_decode_against_plain(wider_folder, "wider", wider_plain, dtype, tol)


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 3e-2)])
def test_mha_model_captured_decode_step_against_plain(mha_folder, mha_plain, dtype, tol):
    _captured_decode_against_plain(mha_folder, "mha", mha_plain, dtype, tol)


def _pieces_against_plain(path, kind, want, dtype, tol):
    """Three sequences whose prompts come in three pieces of unequal sizes: every step after the
    first brings several tokens on top of a past that differs per sequence."""
    import rbitnet_amd
    reqs, want = _tokens(kind, PIECES["lengths"], 31), want["pieces"]
    eng = rbitnet_amd.Engine.load_path(path, dtype=dtype, max_tokens=64 * 10, max_batch=len(reqs))
    for g in eng.cache.kv_groups:
        g.k.fill_(float("nan"))
        g.v.fill_(float("nan"))
    slots = [eng.alloc_slot() for _ in reqs]
    done = [0] * len(reqs)
    got = [[] for _ in reqs]
    for cut in PIECES["cuts"] + [[len(r) for r in reqs]]:
        sizes = [min(c, len(r) - d) for c, r, d in zip(cut, reqs, done)]
        logits = eng.step([(s, r[d:d + n]) for s, r, d, n in zip(slots, reqs, done, sizes)], "all").cpu()
        off = 0
        for i, n in enumerate(sizes):
            got[i].append(logits[off:off + n])
            off += n
            done[i] += n
    assert done == [len(r) for r in reqs]
    for s in slots:
        eng.free_slot(s)
    for i, (r, w) in enumerate(zip(reqs, want)):
        err = (torch.cat(got[i]).double() - w).abs().amax(dim=1) / w.abs().max()
        assert float(err.max()) < tol, f"{kind} {dtype}: request {i}, position {int(err.argmax())}: {float(err.max())}"
    del eng
    torch.cuda.empty_cache()


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 3e-2)])
def test_wide_model_prompts_in_pieces_against_plain(folder, wide_plain, dtype, tol):
    _pieces_against_plain(folder, "wide", wide_plain, dtype, tol)


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 3e-2)])
def test_mha_model_prompts_in_pieces_against_plain(mha_folder, mha_plain, dtype, tol):
    _pieces_against_plain(mha_folder, "mha", mha_plain, dtype, tol)


def test_wide_model_bfloat16_against_float32(folder):
    """A drift report rather than a proof: twenty requests, alone and together, against the
    engine's own float32 path (which the tests above compare with the plain implementation)."""
    import rbitnet_amd
    rng = np.random.default_rng(3)
    lengths = [700, 130, 65, 300, 1, 31, 64, 200, 90, 17, 450, 33, 257, 129, 5, 512, 77, 256, 40, 100]
    prompts = [[int(t) for t in rng.integers(0, 128256, size=n)] for n in lengths]
    tail = 3                                        # tokens of each request that are decoded one by one

    ref = rbitnet_amd.Engine.load_path(folder, dtype="float32", max_tokens=64 * 80, max_batch=len(prompts))
    want = []
    for p in prompts:
        s = ref.alloc_slot()
        rows = list(range(max(0, len(p) - tail - 1), len(p)))
        want.append(ref.step([(s, p)], [rows]).cpu())
        ref.free_slot(s)
    del ref
    torch.cuda.empty_cache()

    eng = rbitnet_amd.Engine.load_path(folder, dtype="bfloat16", max_tokens=64 * 80, max_batch=len(prompts))
    tol = 3e-2
    # (1) each alone: a prompt step (tiled products, flash attention), then single tokens (skinny and
    #     token-resident products, decode attention with splits)
    for p, w in zip(prompts[:6], want[:6]):
        s = eng.alloc_slot()
        head = max(1, len(p) - tail)
        got = [eng.step([(s, p[:head])], "last")]
        for t in p[head:]:
            got.append(eng.step([(s, [t])], "last"))
        eng.free_slot(s)
        got = torch.cat(got).cpu()
        assert _rel(got, w[-got.shape[0]:]) < tol, len(p)
    # (2) all twenty together: one ragged prompt step, then steps of up to 20 single tokens (panel
    #     products) launched kernel by kernel, the requests' last `tail` tokens being fed one by one
    slots = [eng.alloc_slot() for _ in prompts]
    heads = [max(1, len(p) - tail) for p in prompts]
    logits = eng.step([(s, p[:h]) for s, p, h in zip(slots, prompts, heads)], "last").cpu()
    for i, (p, h, w) in enumerate(zip(prompts, heads, want)):
        assert _rel(logits[i:i + 1], w[h - 1 - (len(p) - w.shape[0]):][:1]) < tol, ("prompt", i)
    for j in range(tail):
        live = [i for i, (p, h) in enumerate(zip(prompts, heads)) if h + j < len(p)]
        logits = eng.step([(slots[i], [prompts[i][heads[i] + j]]) for i in live], "last").cpu()
        for r, i in enumerate(live):
            w = want[i]
            pos = heads[i] + j
            assert _rel(logits[r:r + 1], w[pos - (len(prompts[i]) - w.shape[0]):][:1]) < tol, ("decode", i, j)
    for s in slots:
        eng.free_slot(s)
    eng.cache.check()
