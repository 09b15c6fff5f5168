"""Each part alone against the plain functions, and the generality of the composition:
a toy mixer with state of its own, defined here, registered, built and stepped without a
change to the framework; layers of different kinds and sizes in one model; a layer that
runs twice; a layer that reads another layer's cache; a window."""
import math

import pytest
import torch

import plain_llama as P
from rbitnet_amd.cache import Cache
from rbitnet_amd.config.spec import LayerSpec, ModelSpec, PartSpec
from rbitnet_amd.engine.context import StepBatch, StepContext
from rbitnet_amd.parts import BuildEnv, CacheRequest, Part, TensorSpec, build_part, register_mixer

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
D64 = torch.float64


@pytest.fixture(scope="module")
def lib():
    from rbitnet_amd.csrc.lib import kernels
    return kernels()


def _env(lib, hidden, dtype):
    return BuildEnv(hidden_size=hidden, dtype=dtype, device=torch.device(DEV), lib=lib)


def _rel(got, want):
    want = want.double().cpu()
    return float((got.double().cpu() - want).abs().max() / want.abs().max())


def _ctx_and_cache(part, past, tokens_per_seq, dtype):
    """A cache for one mixer and a step context for sequences with `past` tokens already
    stored (the caller fills them by running earlier steps)."""
    cache = Cache([part.cache_request()], len(past), 64 * 16, dtype, DEV)
    slots = [cache.alloc_slot() for _ in past]
    return cache, slots


def _step(cache, slots, q_lens):
    from rbitnet_amd.csrc.lib import kernels
    past = [cache.length(s) for s in slots]
    cache.reserve(slots, q_lens)
    return StepContext.for_batch(DEV, StepBatch(slots, past, [[0] * q for q in q_lens], [], cache.block_tables(slots)),
                                 n_compute_units=kernels().n_compute_units)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-6), (torch.bfloat16, 8e-3)])
def test_norm_part(lib, dtype, tol):
    part = build_part("norm", PartSpec("rmsnorm", {"size": 100, "eps": 1e-3}), _env(lib, 100, dtype))
    assert part.tensor_specs()["weight"].shape == (100,) and part.tensor_specs()["weight"].role == "gain"
    w = 1 + 0.2 * torch.randn(100)
    part.load({"weight": w.to(DEV)})
    x, d = torch.randn(5, 100) * 0.03, torch.randn(5, 100) * 0.03
    xd = x.to(DEV).clone()
    got = part.forward(xd, d.to(DEV))
    assert got.dtype == dtype and _rel(got, P.rmsnorm((x + d).double(), w.double(), 1e-3)) < tol
    assert torch.equal(xd.cpu(), x + d)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-6), (torch.bfloat16, 2e-2)])
def test_feed_forward_part(lib, dtype, tol):
    for hidden, ff in ((40, 52), (64, 96)):              # generic path, then the fused matrix-core path
        part = build_part("feed_forward", PartSpec("swiglu", {"intermediate_size": ff}), _env(lib, hidden, dtype))
        names = part.names
        w = {names["gate"]: torch.randn(ff, hidden) * 0.3, names["up"]: torch.randn(ff, hidden) * 0.3,
             names["down"]: torch.randn(hidden, ff) * 0.3}
        w = {k: v.to(dtype) for k, v in w.items()}
        part.load({k: v.to(DEV) for k, v in w.items()})
        h = torch.randn(7, hidden).to(dtype)
        got = part.forward(h.to(DEV))
        want = P.swiglu(h.double(), w[names["gate"]].double(), w[names["up"]].double(), w[names["down"]].double())
        assert got.dtype == torch.float32 and _rel(got, want) < tol, (hidden, ff)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-6), (torch.bfloat16, 8e-3)])
@pytest.mark.parametrize("style", ["interleaved", "half"])
def test_position_part(lib, dtype, tol, style):
    """The rotation part alone: two sequences on unequal pasts bring unequal pieces; q comes back rotated, the
    rotated k and the plain v lie in the cache at the tokens' positions, with the llama3 rule's three ranges of
    frequencies in play (positions beyond the original 32)."""
    hq, hk, d = 3, 2, 24
    scaling = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
               "original_max_position_embeddings": 32}
    part = build_part("position", PartSpec("rope", {"head_dim": d, "theta": 500000.0, "scaling": scaling, "style": style,
                                                    "max_positions": 512}), _env(lib, 48, dtype))
    cache = Cache([CacheRequest("kv", heads=hk, head_dim=d, window=None)], 2, 64 * 8, dtype, DEV)
    slots = [cache.alloc_slot(), cache.alloc_slot()]
    cache.reserve(slots, [70, 3])
    cache.commit(slots, [70, 3])                       # what lies there already is not read here
    q_lens = [5, 66]
    ctx = _step(cache, slots, q_lens)
    view = cache.view(0, ctx.block_tables)
    n = sum(q_lens)
    qkv = torch.randn(n, (hq + 2 * hk) * d)
    q = torch.empty(n, hq, d, dtype=dtype, device=DEV)
    part.encode_and_store(qkv.to(DEV), q, view.k_pages, view.v_pages, ctx, view.block_table, hq, hk, d)
    inv = P.rope_inv_freq(d, 500000.0, scaling)
    positions = [70 + i for i in range(5)] + [3 + i for i in range(66)]
    seq_of = [0] * 5 + [1] * 66
    tables = cache.block_tables(slots)
    pages = tables[next(iter(tables))]
    kp, vp = view.k_pages.cpu().double(), view.v_pages.cpu().double()
    worst = 0.0
    for t, (pos, b) in enumerate(zip(positions, seq_of)):
        row = qkv[t].double()
        for h in range(hq):
            want = P.rope(row[h * d:(h + 1) * d], pos, inv, style)
            worst = max(worst, float((q[t, h].double().cpu() - want).abs().max() / want.abs().max()))
        page, at = pages[b][pos // 64], pos % 64
        for h in range(hk):
            want_k = P.rope(row[(hq + h) * d:(hq + h + 1) * d], pos, inv, style)
            want_v = row[(hq + hk + h) * d:(hq + hk + h + 1) * d]
            worst = max(worst, float((kp[page, h, at] - want_k).abs().max() / want_k.abs().max()))
            worst = max(worst, float((vp[page, h, at] - want_v).abs().max() / want_v.abs().max().clamp_min(1e-30)))
    assert worst < tol


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-6), (torch.bfloat16, 8e-3)])
@pytest.mark.parametrize("tied", [False, True])
def test_the_two_ends_alone(lib, dtype, tol, tied):
    """The embedding part (rows of the table by token id) and the head part (the final norm and the output
    matrix on the asked rows only, with a pending term still to be added; tied: the embedding's table)."""
    hidden, vocab = 40, 333
    env = _env(lib, hidden, dtype)
    emb = build_part("embedding", PartSpec("table", {"name": "emb.weight", "vocab_size": vocab}), env)
    head = build_part("head", PartSpec("linear", {"norm": PartSpec("rmsnorm", {"size": hidden, "eps": 1e-4}),
                                                  "norm_name": "final.weight", "name": None if tied else "out.weight",
                                                  "vocab_size": vocab}), env)
    assert set(emb.tensor_specs()) == {"emb.weight"}
    assert set(head.tensor_specs()) == ({"final.weight"} if tied else {"final.weight", "out.weight"})
    table = (torch.randn(vocab, hidden) * 0.5).to(dtype)
    out_w = (torch.randn(vocab, hidden) * 0.5).to(dtype)
    gain = 1 + 0.2 * torch.randn(hidden)
    emb.load({"emb.weight": table.to(DEV)})
    head.load({"final.weight": gain.to(DEV), "out.weight": out_w.to(DEV)}, embedding=emb)
    ids = [5, 332, 0, 17, 17, 200, 9]
    ctx = StepContext.for_batch(DEV, StepBatch([0, 1], [0, 0], [ids[:4], ids[4:]], [3, 6], {}),
                                n_compute_units=lib.n_compute_units)
    x = emb.forward(ctx)
    assert x.dtype == torch.float32 and torch.equal(x.cpu(), table[ids].float())
    pending = (torch.randn(len(ids), hidden) * 0.3).to(DEV)
    want_rows = (x.cpu().double() + pending.cpu().double())[[3, 6]]
    logits = head.forward(x, pending, ctx.rows, ctx)
    w = (table if tied else out_w).double()
    want = P.linear(P.rmsnorm(want_rows, gain.double(), 1e-4), w)
    assert logits.dtype == torch.float32 and logits.shape == (2, vocab)
    assert _rel(logits, want) < tol
    from rbitnet_amd.errors import ConfigError
    if tied:
        with pytest.raises(ConfigError, match="share"):
            head.load({"final.weight": gain.to(DEV)}, embedding=None)


def _attention_params(hq, hk, d, window=None, theta=10000.0, style="interleaved", scaling=None):
    return {"num_heads": hq, "num_kv_heads": hk, "head_dim": d, "scale": 1 / math.sqrt(d), "window": window,
            "cache_from": None,
            "position": PartSpec("rope", {"head_dim": d, "theta": theta, "scaling": scaling, "style": style,
                                          "max_positions": 512})}


def _plain_attention_layer(h, w, names, hq, hk, d, theta, style, window):
    q, k, v = (P.linear(h, w[names[n]].double()) for n in ("q", "k", "v"))
    inv = P.rope_inv_freq(d, theta, None)
    for pos in range(h.shape[0]):
        for i in range(hq):
            q[pos, i * d:(i + 1) * d] = P.rope(q[pos, i * d:(i + 1) * d], pos, inv, style)
        for i in range(hk):
            k[pos, i * d:(i + 1) * d] = P.rope(k[pos, i * d:(i + 1) * d], pos, inv, style)
    return P.linear(P.attention(q, k, v, hq, hk, window), w[names["o"]].double())


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 3e-6), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("hq,hk,d,window,style", [(6, 3, 10, None, "interleaved"), (4, 1, 64, None, "half"),
                                                  (8, 2, 128, 50, "interleaved"), (2, 2, 32, 7, "half")])
def test_attention_part_whole_and_in_pieces(lib, dtype, tol, hq, hk, d, window, style):
    hidden = 48
    part = build_part("mixer", PartSpec("attention", _attention_params(hq, hk, d, window, style=style)),
                      _env(lib, hidden, dtype))
    specs = part.tensor_specs()
    w = {n: (torch.randn(s.shape) * 0.2).to(dtype) for n, s in specs.items()}
    part.load({n: t.to(DEV) for n, t in w.items()})
    t_len = 150
    h = torch.randn(t_len, hidden).to(dtype)
    want = _plain_attention_layer(h.double(), w, part.names, hq, hk, d, 10000.0, style, window)
    for cuts in ([t_len], [100, 1, 1, 48], [64, 64, 22]):
        cache, slots = _ctx_and_cache(part, [0], None, dtype)
        outs, at = [], 0
        for n in cuts:
            ctx = _step(cache, slots, [n])
            view = cache.view(0, ctx.block_tables)
            outs.append(part.forward(h[at:at + n].to(DEV).contiguous(), ctx, view))
            cache.commit(slots, [n])
            at += n
        assert _rel(torch.cat(outs), want) < tol, cuts


# ---------------------------------------------------------------------------- a toy mixer with state
class DecayMixer(Part):
    """s_t = a * s_{t-1} + h_t per sequence (a fixed-size state, no keys or values),
    out_t = W s_t.  Written with torch operations: the framework only has to hand it its
    state and the batch's layout."""

    def __init__(self, params, env):
        self.env, self.a, self.hidden = env, float(params["decay"]), env.hidden_size

    def tensor_specs(self):
        return {"mix.weight": TensorSpec((self.hidden, self.hidden))}

    def load(self, tensors):
        self.w = tensors["mix.weight"]

    def cache_request(self):
        return CacheRequest("state", state_shape=(self.hidden,), state_init=0.0)

    def forward(self, h, ctx, view):
        hf = h.float()
        out = torch.empty_like(hf)
        cu = ctx.cu_seqlens.tolist()
        for b, slot in enumerate(ctx.host_slots):
            s = view.state[slot]
            for t in range(cu[b], cu[b + 1]):
                s = self.a * s + hf[t]
                out[t] = s
            view.state[slot] = s
        return out @ self.w.float().T


def _plain_toy_model(spec, tensors, tokens):
    """The hand-made model of test_toy_mixer... computed plainly in float64."""
    w = {k: v.double().cpu() for k, v in tensors.items()}
    x = P.embedding(w[spec.embedding_name], tokens)
    states = {}
    for place, i in enumerate(spec.schedule):
        layer = spec.layers[i]
        pre = layer.prefix
        h = P.rmsnorm(x, w[f"{pre}.input_layernorm.weight"], layer.norm1["eps"])
        if layer.mixer.kind == "toy_decay":
            s = torch.zeros(spec.hidden_size, dtype=D64)
            rows = []
            for t in range(h.shape[0]):
                s = layer.mixer["decay"] * s + h[t]
                rows.append(s)
            a = P.linear(torch.stack(rows), w[f"{pre}.self_attn.mix.weight"])
            states[place] = None
        else:
            m = layer.mixer
            hq, hk, d = m["num_heads"], m["num_kv_heads"], m["head_dim"]
            inv = P.rope_inv_freq(d, m["position"]["theta"], None)
            q = P.linear(h, w[f"{pre}.self_attn.q_proj.weight"])
            for pos in range(h.shape[0]):
                for j in range(hq):
                    q[pos, j * d:(j + 1) * d] = P.rope(q[pos, j * d:(j + 1) * d], pos, inv)
            if m["cache_from"] is None:
                k = P.linear(h, w[f"{pre}.self_attn.k_proj.weight"])
                v = P.linear(h, w[f"{pre}.self_attn.v_proj.weight"])
                for pos in range(h.shape[0]):
                    for j in range(hk):
                        k[pos, j * d:(j + 1) * d] = P.rope(k[pos, j * d:(j + 1) * d], pos, inv)
                states[place] = (k, v)
            else:
                src = [p for p in range(place) if spec.schedule[p] == m["cache_from"]][-1]
                k, v = states[src]
            a = P.linear(P.attention(q, k, v, hq, hk, m["window"]), w[f"{pre}.self_attn.o_proj.weight"])
        x = x + a
        h2 = P.rmsnorm(x, w[f"{pre}.post_attention_layernorm.weight"], layer.norm2["eps"])
        x = x + P.swiglu(h2, w[f"{pre}.mlp.gate_proj.weight"], w[f"{pre}.mlp.up_proj.weight"],
                         w[f"{pre}.mlp.down_proj.weight"])
    xn = P.rmsnorm(x, w[spec.final_norm_name], spec.final_norm["eps"])
    return P.linear(xn, w[spec.head_name])


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 3e-2)])
def test_toy_mixer_and_mixed_layers(dtype, tol):
    """Layer 0: windowed attention.  Layer 1: the toy state mixer with a wider
    feed-forward.  Layer 2: attention that reads layer 0's cache, other eps.  Schedule
    0, 1, 2, 1: layer 1 runs twice, with a state per run."""
    import rbitnet_amd
    from rbitnet_amd.engine.model import expected_tensors
    from rbitnet_amd.weights import random_tensors
    register_mixer("toy_decay", DecayMixer)
    hidden, vocab = 48, 90
    norm = lambda eps: PartSpec("rmsnorm", {"size": hidden, "eps": eps})
    att0 = _attention_params(4, 2, 16, window=40)
    att2 = dict(_attention_params(4, 2, 16, window=33), cache_from=0)
    layers = [
        LayerSpec("blocks.0", "prenorm", PartSpec("attention", att0), PartSpec("swiglu", {"intermediate_size": 64}),
                  norm(1e-5), norm(1e-5)),
        LayerSpec("blocks.1", "prenorm", PartSpec("toy_decay", {"decay": 0.7}),
                  PartSpec("swiglu", {"intermediate_size": 100}), norm(1e-5), norm(1e-5)),
        LayerSpec("blocks.2", "prenorm", PartSpec("attention", att2), PartSpec("swiglu", {"intermediate_size": 32}),
                  norm(1e-3), norm(1e-3)),
    ]
    spec = ModelSpec(architecture="ToyForTests", hidden_size=hidden, vocab_size=vocab, max_positions=512,
                     embedding_name="embed.weight", layers=layers, final_norm=norm(1e-5),
                     final_norm_name="final_norm.weight", head_name="head.weight", schedule=[0, 1, 2, 1])
    # a reader must not look further back than the cache it reads keeps
    bad = ModelSpec(architecture="ToyForTests", hidden_size=hidden, vocab_size=vocab, max_positions=512,
                    embedding_name="embed.weight", final_norm=norm(1e-5), final_norm_name="final_norm.weight",
                    head_name="head.weight", layers=[layers[0], LayerSpec(
                        "blocks.1", "prenorm", PartSpec("attention", dict(att2, window=None)),
                        PartSpec("swiglu", {"intermediate_size": 32}), norm(1e-5), norm(1e-5))])
    from rbitnet_amd.engine.model import Model
    from rbitnet_amd.errors import ConfigError
    with pytest.raises(ConfigError, match="keeps only the last 40"):
        Model(bad, torch.float32, DEV, None).cache_readers()
    expected = expected_tensors(spec)
    assert "blocks.1.self_attn.mix.weight" in expected and "blocks.2.self_attn.k_proj.weight" not in expected
    tensors = dict(random_tensors(expected, seed=4, std=0.15, norm_std=0.05, dtype=torch.bfloat16))
    eng = rbitnet_amd.Engine.from_spec(spec, tensors, dtype=dtype, max_tokens=64 * 12, max_batch=3)
    assert len(eng.cache.kv_groups) == 1 and len(eng.cache.state_groups) == 1
    assert eng.cache.state_groups[0].data.shape[:2] == (2, 3 + 1)  # two runs of layer 1, two states; 3 slots and the spare one
    g = torch.Generator().manual_seed(8)
    seqs = [torch.randint(0, vocab, (n,), generator=g).tolist() for n in (130, 9, 70)]
    want = [_plain_toy_model(spec, tensors, s) for s in seqs]
    # whole
    for s, w in zip(seqs, want):
        slot = eng.alloc_slot()
        assert _rel(eng.step([(slot, s)], "all"), w) < tol
        eng.free_slot(slot)
    # as a batch: unequal prompts, then one token each; slots used again (state must be reset)
    slots = [eng.alloc_slot() for _ in seqs]
    cut = [len(s) - 5 for s in seqs]
    logits = eng.step([(sl, s[:c]) for sl, s, c in zip(slots, seqs, cut)], "all")
    off = 0
    for s, c, w in zip(seqs, cut, want):
        assert _rel(logits[off:off + c], w[:c]) < tol
        off += c
    for j in range(5):
        logits = eng.step([(sl, [s[c + j]]) for sl, s, c in zip(slots, seqs, cut)], "last")
        for i, (c, w) in enumerate(zip(cut, want)):
            assert _rel(logits[i:i + 1], w[c + j:c + j + 1]) < tol * 2
    for sl in slots:
        eng.free_slot(sl)
    eng.cache.check()
    # the windowed group gave pages back while the long sequence ran
    assert eng.cache.kv_groups[0].table.pool.n_free == eng.cache.n_pages


class ScaledDecayMixer(Part):
    """The state mixer again, with two things more: its input is weighted per token by an array
    that the step layout carries for it (declared below with `declare_step_array`, computed on the
    host from the batch for every step), and with one token per sequence its forward only launches
    device work, so that the decode step it is part of can be captured:
        s_t = a * s_{t-1} + h_t / (1 + pos_t / 8),  out_t = W s_t."""
    graph_safe = True

    def __init__(self, params, env):
        self.env, self.a, self.hidden = env, float(params["decay"]), env.hidden_size

    def tensor_specs(self):
        return {"mix.weight": TensorSpec((self.hidden, self.hidden))}

    def load(self, tensors):
        self.w = tensors["mix.weight"]

    def cache_request(self):
        return CacheRequest("state", state_shape=(self.hidden,), state_init=0.0)

    def forward(self, h, ctx, view):
        hf = h.float() * ctx.extra["toy_token_weight"][:, None]
        if ctx.max_q_len == 1:                               # one token each: device work only
            idx = ctx.slots.long()
            s = self.a * view.state.index_select(0, idx) + hf
            view.state.index_copy_(0, idx, s)
            return s @ self.w.float().T
        out = torch.empty_like(hf)
        at = 0
        for slot, n in zip(ctx.host_slots, ctx.q_lens):      # the host knows the layout: nothing is read back
            s = view.state[slot]
            for t in range(at, at + n):
                s = self.a * s + hf[t]
                out[t] = s
            view.state[slot] = s
            at += n
        return out @ self.w.float().T


def _toy_token_weight(batch):
    import numpy as np
    pos = np.concatenate([p + np.arange(len(t)) for p, t in zip(batch.past_lens, batch.tokens)])
    return (1.0 / (1.0 + pos / 8.0)).astype(np.float32)


def test_toy_mixer_with_a_step_array_of_its_own_runs_captured():
    """One declaration gives a part a per-step array, in steps launched kernel by kernel and in the
    captured decode step alike; the state is updated once per step there too (the step that runs
    before the capture counts, the capture itself executes nothing)."""
    import rbitnet_amd
    from rbitnet_amd.engine.context import declare_step_array, forget_step_array
    declare_step_array("toy_token_weight", "float32", lambda n_seqs, n_tokens: n_tokens, _toy_token_weight)
    try:
        _run_scaled_decay_model()
    finally:
        forget_step_array("toy_token_weight")


def _run_scaled_decay_model():
    import rbitnet_amd
    from rbitnet_amd.engine.model import expected_tensors
    from rbitnet_amd.weights import random_tensors
    register_mixer("toy_scaled_decay", ScaledDecayMixer)
    hidden, vocab = 64, 80
    norm = PartSpec("rmsnorm", {"size": hidden, "eps": 1e-5})
    layers = [LayerSpec(f"blocks.{i}", "prenorm", PartSpec("toy_scaled_decay", {"decay": 0.6 + 0.1 * i}),
                        PartSpec("swiglu", {"intermediate_size": 96}), norm, norm) for i in range(2)]
    spec = ModelSpec(architecture="ToyForTests", hidden_size=hidden, vocab_size=vocab, max_positions=256,
                     embedding_name="embed.weight", layers=layers, final_norm=norm,
                     final_norm_name="final_norm.weight", head_name="head.weight")
    tensors = dict(random_tensors(expected_tensors(spec), seed=9, std=0.2, norm_std=0.05, dtype=torch.bfloat16))

    def plain(tokens):
        w = {k: v.double() for k, v in tensors.items()}
        x = P.embedding(w["embed.weight"], tokens)
        for i, layer in enumerate(spec.layers):
            pre = layer.prefix
            h = P.rmsnorm(x, w[f"{pre}.input_layernorm.weight"], 1e-5)
            s, rows = torch.zeros(hidden, dtype=D64), []
            for t in range(h.shape[0]):
                s = layer.mixer["decay"] * s + h[t] / (1.0 + t / 8.0)
                rows.append(s)
            x = x + P.linear(torch.stack(rows), w[f"{pre}.self_attn.mix.weight"])
            h2 = P.rmsnorm(x, w[f"{pre}.post_attention_layernorm.weight"], 1e-5)
            x = x + P.swiglu(h2, w[f"{pre}.mlp.gate_proj.weight"], w[f"{pre}.mlp.up_proj.weight"],
                             w[f"{pre}.mlp.down_proj.weight"])
        return P.linear(P.rmsnorm(x, w["final_norm.weight"], 1e-5), w["head.weight"])

    eng = rbitnet_amd.Engine.from_spec(spec, tensors, dtype="float32", max_tokens=64 * 4, max_batch=2)
    assert eng.use_graphs and not eng.cache.kv_groups
    g = torch.Generator().manual_seed(3)
    seqs = [torch.randint(0, vocab, (n,), generator=g).tolist() for n in (30, 12)]
    want = [plain(s) for s in seqs]
    for graphs in (True, False):
        eng.use_graphs = graphs
        slots = [eng.alloc_slot() for _ in seqs]
        cut = [len(s) - 6 for s in seqs]
        logits = eng.step([(sl, s[:c]) for sl, s, c in zip(slots, seqs, cut)], "last")
        for i, (c, w) in enumerate(zip(cut, want)):
            assert _rel(logits[i:i + 1], w[c - 1:c]) < 2e-5
        for j in range(6):                                   # decode steps: the first runs before the capture
            eng.decode_step(slots, [s[c + j] for s, c in zip(seqs, cut)])
            for i, (c, w) in enumerate(zip(cut, want)):
                assert _rel(eng.last_decode_logits[i:i + 1], w[c + j:c + j + 1]) < 2e-5, (graphs, j, i)
        for sl in slots:
            eng.free_slot(sl)
    assert len(eng._graphs) == 1


# ---------------------------------------------------------------------------- other toy parts
class HalfRotary(Part):
    """Another position encoding, defined here: only the first half of each head's pairs is
    rotated (the rest keeps angle 0), with frequencies of its own.  It is nothing but
    another angle table for the existing kernels, the fused decode kernel included."""
    graph_safe = True

    def __init__(self, params, env):
        self.env = env
        d = int(params["head_dim"])
        n = int(params["max_positions"])
        inv = torch.zeros(d // 2, dtype=torch.float64)
        inv[: d // 4] = 1.0 / (float(params["theta"]) ** (torch.arange(d // 4, dtype=torch.float64) * 4 / d))
        self.inv = inv
        ang = torch.arange(n, dtype=torch.float64)[:, None] * inv[None, :]
        self.cos = torch.cos(ang).float().to(env.device) if env.lib is not None else None
        self.sin = torch.sin(ang).float().to(env.device) if env.lib is not None else None

    def rotation_tables(self):
        return self.cos, self.sin, 0

    def encode_and_store(self, qkv, q_out, k_pages, v_pages, ctx, block_table, n_heads, n_kv, head_dim):
        self.env.lib.rope_kv_write(qkv, self.cos, self.sin, 0, q_out, k_pages, v_pages, ctx.tok_pos, ctx.tok_seq,
                                   block_table, n_heads, n_kv, head_dim)


class TopOneExperts(Part):
    """A feed-forward with routing, defined here: a float32 router picks one of E small
    SiLU-gated experts per token (torch operations; scratch sized by the step's tokens)."""

    def __init__(self, params, env):
        self.env, self.n_exp, self.ff, self.hidden = env, int(params["experts"]), int(params["ff"]), env.hidden_size

    def tensor_specs(self):
        specs = {"router.weight": TensorSpec((self.n_exp, self.hidden), role="gain", init="normal")}
        for e in range(self.n_exp):
            specs[f"experts.{e}.gate.weight"] = TensorSpec((self.ff, self.hidden))
            specs[f"experts.{e}.up.weight"] = TensorSpec((self.ff, self.hidden))
            specs[f"experts.{e}.down.weight"] = TensorSpec((self.hidden, self.ff))
        return specs

    def load(self, tensors):
        self.w = tensors

    def forward(self, h, ctx=None):
        hf = h.float()
        choice = (hf @ self.w["router.weight"].float().T).argmax(dim=1)
        out = torch.zeros_like(hf)
        for e in range(self.n_exp):
            rows = (choice == e).nonzero().flatten()
            if rows.numel():
                x = hf[rows]
                g = x @ self.w[f"experts.{e}.gate.weight"].float().T
                u = x @ self.w[f"experts.{e}.up.weight"].float().T
                out[rows] = (torch.nn.functional.silu(g) * u) @ self.w[f"experts.{e}.down.weight"].float().T
        return out


def _plain_other_parts(spec, tensors, tokens, inv):
    w = {k: v.double().cpu() for k, v in tensors.items()}
    x = P.embedding(w[spec.embedding_name], tokens)
    margin = float("inf")
    for layer in spec.layers:
        pre = layer.prefix
        m = layer.mixer
        hq, hk, d = m["num_heads"], m["num_kv_heads"], m["head_dim"]
        h = P.rmsnorm(x, w[f"{pre}.input_layernorm.weight"], layer.norm1["eps"])
        q = P.linear(h, w[f"{pre}.self_attn.q_proj.weight"])
        k = P.linear(h, w[f"{pre}.self_attn.k_proj.weight"])
        v = P.linear(h, w[f"{pre}.self_attn.v_proj.weight"])
        for pos in range(h.shape[0]):
            for j in range(hq):
                q[pos, j * d:(j + 1) * d] = P.rope(q[pos, j * d:(j + 1) * d], pos, inv)
            for j in range(hk):
                k[pos, j * d:(j + 1) * d] = P.rope(k[pos, j * d:(j + 1) * d], pos, inv)
        x = x + P.linear(P.attention(q, k, v, hq, hk, None), w[f"{pre}.self_attn.o_proj.weight"])
        h2 = P.rmsnorm(x, w[f"{pre}.post_attention_layernorm.weight"], layer.norm2["eps"])
        logits = P.linear(h2, w[f"{pre}.mlp.router.weight"])
        f = torch.zeros_like(x)
        top = torch.topk(logits, 2, dim=1).values
        margin = min(margin, float((top[:, 0] - top[:, 1]).min()))
        for t in range(x.shape[0]):
            e = int(logits[t].argmax())
            f[t] = P.swiglu(h2[t:t + 1], w[f"{pre}.mlp.experts.{e}.gate.weight"], w[f"{pre}.mlp.experts.{e}.up.weight"],
                            w[f"{pre}.mlp.experts.{e}.down.weight"])[0]
        x = x + f
    xn = P.rmsnorm(x, w[spec.final_norm_name], spec.final_norm["eps"])
    return P.linear(xn, w[spec.head_name]), margin


def test_toy_position_and_routed_feed_forward():
    """Registered from the test, built by the framework, stepped whole, in pieces and as a
    batch; head size 64 so that the matrix-core attention kernels (and the fused decode
    kernel with the toy's angle table) run."""
    import rbitnet_amd
    from rbitnet_amd.engine.model import expected_tensors
    from rbitnet_amd.parts import register_feed_forward, register_position
    from rbitnet_amd.weights import random_tensors
    register_position("half_rotary", HalfRotary)
    register_feed_forward("top_one_experts", TopOneExperts)
    hidden, vocab, d = 64, 70, 64
    norm = PartSpec("rmsnorm", {"size": hidden, "eps": 1e-5})
    pos = PartSpec("half_rotary", {"head_dim": d, "theta": 100.0, "max_positions": 512})
    att = {"num_heads": 2, "num_kv_heads": 1, "head_dim": d, "scale": d ** -0.5, "window": None, "cache_from": None,
           "position": pos}
    layers = [LayerSpec(f"blocks.{i}", "prenorm", PartSpec("attention", att),
                        PartSpec("top_one_experts", {"experts": 3, "ff": 40}), norm, norm) for i in range(2)]
    spec = ModelSpec(architecture="ToyForTests", hidden_size=hidden, vocab_size=vocab, max_positions=512,
                     embedding_name="embed.weight", layers=layers, final_norm=norm,
                     final_norm_name="final_norm.weight", head_name="head.weight")
    expected = expected_tensors(spec)
    assert "blocks.1.mlp.experts.2.down.weight" in expected
    tensors = dict(random_tensors(expected, seed=6, std=0.15, norm_std=0.05, dtype=torch.bfloat16))
    for name in tensors:
        if name.endswith("router.weight"):
            tensors[name] = tensors[name] * 8          # clear-cut choices, so that rounding cannot flip one
    eng = rbitnet_amd.Engine.from_spec(spec, tensors, dtype="bfloat16", max_tokens=64 * 8, max_batch=2)
    assert not eng.use_graphs                          # the routed feed-forward reads device data on the host
    inv = HalfRotary(pos.params, BuildEnv(hidden, torch.float32, torch.device("cpu"), None)).inv
    # a router's choice between two nearly equal logits may fall either way in bfloat16: take
    # sequences whose choices are all clear-cut in the plain computation
    g = torch.Generator().manual_seed(2)
    seqs, want = [], []
    for n in (90, 20):
        for _ in range(20):
            s = torch.randint(0, vocab, (n,), generator=g).tolist()
            logits, margin = _plain_other_parts(spec, tensors, s, inv)
            if margin > 0.15:
                break
        else:
            pytest.fail("no sequence with clear-cut routing found")
        seqs.append(s)
        want.append(logits)
    slots = [eng.alloc_slot() for _ in seqs]
    cut = [len(s) - 4 for s in seqs]
    logits = eng.step([(sl, s[:c]) for sl, s, c in zip(slots, seqs, cut)], "all")
    off = 0
    for s, c, w in zip(seqs, cut, want):
        assert _rel(logits[off:off + c], w[:c]) < 4e-2
        off += c
    for j in range(4):
        logits = eng.step([(sl, [s[c + j]]) for sl, s, c in zip(slots, seqs, cut)], "last")
        for i, (c, w) in enumerate(zip(cut, want)):
            assert _rel(logits[i:i + 1], w[c + j:c + j + 1]) < 4e-2
    for sl in slots:
        eng.free_slot(sl)


class ScaledTable(Part):
    """An embedding of the test's own: the row of the table times a constant (as architectures
    that multiply their embeddings by sqrt(width) do)."""
    graph_safe = True

    def __init__(self, params, env):
        self.env, self.name, self.vocab, self.scale = env, params["name"], int(params["vocab_size"]), float(params["scale"])

    def tensor_specs(self):
        return {self.name: TensorSpec((self.vocab, self.env.hidden_size))}

    def load(self, tensors):
        self.table = tensors[self.name]

    def step_bytes(self, element_size):
        return 0

    def forward(self, ctx):
        return self.table.float().index_select(0, ctx.token_ids.long()) * self.scale


class CappedHead(Part):
    """A head of the test's own: no sharing with the embedding, a norm of its own kind and name,
    and logits squeezed into (-cap, cap): cap * tanh(W norm(x) / cap)."""
    graph_safe = True

    def __init__(self, params, env):
        self.env, self.cap, self.vocab = env, float(params["cap"]), int(params["vocab_size"])
        self.norm = build_part("norm", params["norm"], env)

    @property
    def first_norm(self):
        return self.norm

    def tensor_specs(self):
        return {"out.norm.weight": self.norm.tensor_specs()["weight"],
                "out.proj.weight": TensorSpec((self.vocab, self.env.hidden_size))}

    def load(self, tensors, embedding=None):
        self.norm.load({"weight": tensors["out.norm.weight"]})
        self.w = tensors["out.proj.weight"]

    def forward(self, x, pending, rows, ctx=None):
        from rbitnet_amd.parts.linear import linear
        from rbitnet_amd.parts.stream import normed_for
        z = linear(self.env.lib, normed_for(None, self.norm, x, pending, rows), self.w, torch.float32)
        return self.cap * torch.tanh(z / self.cap)


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 3e-2)])
def test_embedding_with_a_scale_and_capped_head_registered_from_here(dtype, tol):
    """The two ends of a model are parts like the others: another embedding and another head are
    registered here, named in a hand-made spec and run by the engine's step and its captured
    decode step, with no change to the package."""
    import rbitnet_amd
    from rbitnet_amd.engine.model import expected_tensors
    from rbitnet_amd.parts import register_embedding, register_head
    from rbitnet_amd.weights import random_tensors
    register_embedding("scaled_table", ScaledTable)
    register_head("capped", CappedHead)
    hidden, vocab, scale = 64, 75, 3.5
    norm = PartSpec("rmsnorm", {"size": hidden, "eps": 1e-5})
    att = _attention_params(4, 2, 16, window=None)
    layers = [LayerSpec(f"blocks.{i}", "prenorm", PartSpec("attention", att), PartSpec("swiglu", {"intermediate_size": 48}),
                        norm, norm) for i in range(2)]
    make_spec = lambda cap: ModelSpec(
        architecture="ToyForTests", hidden_size=hidden, vocab_size=vocab, max_positions=256, layers=layers,
        embedding=PartSpec("scaled_table", {"name": "tokens.weight", "vocab_size": vocab, "scale": scale}),
        head=PartSpec("capped", {"norm": norm, "vocab_size": vocab, "cap": cap}))
    expected = expected_tensors(make_spec(1.0))
    assert {"tokens.weight", "out.norm.weight", "out.proj.weight"} <= set(expected)
    tensors = dict(random_tensors(expected, seed=9, std=0.15, norm_std=0.05, dtype=torch.bfloat16))

    def plain(tokens, cap):
        # the plain Llama layers between the test's own ends
        w = {k: v.double().cpu() for k, v in tensors.items()}
        x = P.embedding(w["tokens.weight"], tokens) * scale
        for i in range(2):
            pre = f"blocks.{i}"
            h = P.rmsnorm(x, w[f"{pre}.input_layernorm.weight"], 1e-5)
            inv = P.rope_inv_freq(16, att["position"]["theta"], None)
            q, k, v = (P.linear(h, w[f"{pre}.self_attn.{n}_proj.weight"]) for n in "qkv")
            q, k = P.rope_rows(q, 4, inv), P.rope_rows(k, 2, inv)
            x = x + P.linear(P.attention(q, k, v, 4, 2), w[f"{pre}.self_attn.o_proj.weight"])
            h2 = P.rmsnorm(x, w[f"{pre}.post_attention_layernorm.weight"], 1e-5)
            x = x + P.swiglu(h2, w[f"{pre}.mlp.gate_proj.weight"], w[f"{pre}.mlp.up_proj.weight"],
                             w[f"{pre}.mlp.down_proj.weight"])
        z = P.linear(P.rmsnorm(x, w["out.norm.weight"], 1e-5), w["out.proj.weight"])
        return z if cap is None else cap * torch.tanh(z / cap)

    g = torch.Generator().manual_seed(12)
    seqs = [torch.randint(0, vocab, (n,), generator=g).tolist() for n in (70, 12)]
    cap = float(plain(seqs[0], None).abs().max()) / 2                     # a cap that bends the large logits
    want = [plain(s, cap) for s in seqs]
    assert float(want[0].abs().max()) > 0.9 * cap
    eng = rbitnet_amd.Engine.from_spec(make_spec(cap), tensors, dtype=dtype, max_tokens=64 * 4, max_batch=2)
    assert eng.use_graphs
    slots = [eng.alloc_slot() for _ in seqs]
    cut = [len(s) - 4 for s in seqs]
    logits = eng.step([(sl, s[:c]) for sl, s, c in zip(slots, seqs, cut)], "all")
    off = 0
    for c, w in zip(cut, want):
        assert _rel(logits[off:off + c], w[:c]) < tol
        off += c
    for j in range(4):                                                    # the captured decode step
        eng.decode_step(slots, [s[c + j] for s, c in zip(seqs, cut)])
        for i, (c, w) in enumerate(zip(cut, want)):
            assert _rel(eng.last_decode_logits[i:i + 1], w[c + j:c + j + 1]) < tol
    assert len(eng._graphs) == 1
    # what a step reads: every tensor of the blocks, the head's two, nothing of the table
    esize = 4 if dtype == "float32" else 2
    per_layer = (64 * 64 * 2 + 2 * 32 * 64 + 3 * 48 * 64) * esize + 2 * 64 * 4
    assert eng.model.weight_bytes() == 2 * per_layer + vocab * hidden * esize + hidden * 4
