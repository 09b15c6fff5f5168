"""The plain implementation pinned by what fixes it beside the reference's text: the
reference's own vectors, special cases that reduce to a library routine, and
invariants.  Each test is chosen so that a plausible mistake (a wrong sign or pairing, a
norm in the wrong place, a mask off by one) fails it.  No GPU."""
import copy
import math

import pytest
import torch
import torch.nn.functional as F

import plain_llama as P
from helpers import model_folder

torch.manual_seed(0)
D64 = torch.float64


def test_linear_reference_vectors():
    # crates/bitnet-core/src/kernels.rs:35-40 and tests/golden_kernels.rs:12-18
    y = P.linear(torch.tensor([[2., 3.]], dtype=D64), torch.tensor([[1., 0.], [-1., 1.]], dtype=D64))
    assert torch.allclose(y, torch.tensor([[2., 1.]], dtype=D64), atol=1e-6)
    w = torch.tensor([[1, -1, 0, 1], [0, 1, 1, -1], [1, 0, -1, 0]], dtype=D64)
    y = P.linear(torch.tensor([[0.5, -0.25, 2.0, 1.0]], dtype=D64), w)
    assert torch.allclose(y, torch.tensor([[1.75, 0.75, -1.5]], dtype=D64), atol=1e-5)
    x, w = torch.randn(4, 7, dtype=D64), torch.randn(5, 7, dtype=D64)
    assert torch.allclose(P.linear(x, w), F.linear(x, w))


def test_embedding():
    t = torch.randn(10, 4, dtype=D64)
    assert torch.equal(P.embedding(t, [3, 0, 9]), F.embedding(torch.tensor([3, 0, 9]), t))
    with pytest.raises(ValueError):
        P.embedding(t, [10])


def test_rmsnorm():
    x, w = torch.randn(3, 33, dtype=D64), torch.randn(33, dtype=D64)
    assert torch.allclose(P.rmsnorm(x, w, 1e-5), F.rms_norm(x, (33,), w, 1e-5))
    c = 0.003
    y = P.rmsnorm(torch.full((1, 8), c, dtype=D64), torch.ones(8, dtype=D64), 1e-5)
    assert torch.allclose(y, torch.full((1, 8), c / math.sqrt(c * c + 1e-5), dtype=D64))
    # eps inside the root, added to the mean: at this scale the alternatives differ by far
    outside = c / (math.sqrt(c * c) + 1e-5)
    assert abs(float(y[0, 0]) - outside) > 0.1
    assert abs(float(P.rmsnorm(torch.full((1, 8), c, dtype=D64), torch.ones(8, dtype=D64), 1e-6)[0, 0])
               - float(y[0, 0])) > 0.1
    big = torch.randn(1, 16, dtype=D64) * 100
    assert torch.allclose(P.rmsnorm(big, w[:16], 1e-5), P.rmsnorm(3 * big, w[:16], 1e-5), atol=1e-8)


def test_softmax_and_silu():
    s = torch.randn(9, dtype=D64) * 5
    assert torch.allclose(P.softmax(s), torch.softmax(s, 0))
    assert torch.allclose(P.softmax(s + 1000.0), P.softmax(s))
    assert torch.isfinite(P.softmax(torch.tensor([1e4, -1e4, 0.0], dtype=D64))).all()
    v = torch.randn(20, dtype=D64) * 4
    assert torch.allclose(P.silu(v), F.silu(v))
    assert float(P.silu(torch.tensor([0.0], dtype=D64))) == 0.0
    assert abs(float(P.silu(torch.tensor([40.0], dtype=D64))) - 40.0) < 1e-9


def test_rope_is_a_complex_rotation_of_adjacent_pairs():
    d = 16
    inv = P.rope_inv_freq(d, 10000.0, None)
    assert float(inv[0]) == 1.0 and torch.all(inv[1:] < inv[:-1])
    x = torch.randn(d, dtype=D64)
    assert torch.equal(P.rope(x, 0, inv), x)                                    # position 0 is the identity
    for pos in (1, 7, 100):
        z = torch.polar(torch.ones(d // 2, dtype=D64), pos * inv)
        want = torch.view_as_real(torch.view_as_complex(x.view(d // 2, 2)) * z).reshape(d)
        assert torch.allclose(P.rope(x, pos, inv), want)                        # sign and pairing
        got = P.rope(x, pos, inv).view(d // 2, 2)
        assert torch.allclose(got.norm(dim=1), x.view(d // 2, 2).norm(dim=1))   # each pair keeps its norm
    # only distances count
    q, k = torch.randn(d, dtype=D64), torch.randn(d, dtype=D64)
    a = (P.rope(q, 9, inv) * P.rope(k, 4, inv)).sum()
    b = (P.rope(q, 59, inv) * P.rope(k, 54, inv)).sum()
    assert abs(float(a - b)) < 1e-9
    assert abs(float(a - (P.rope(q, 10, inv) * P.rope(k, 4, inv)).sum())) > 1e-6


def test_half_style_equals_interleaved_with_permuted_rows():
    d = 12
    inv = P.rope_inv_freq(d, 500.0, None)
    x = torch.randn(d, dtype=D64)
    perm = torch.cat([torch.arange(0, d, 2), torch.arange(1, d, 2)])            # interleaved -> half order
    assert torch.allclose(P.rope(x[perm], 5, inv, "half"), P.rope(x, 5, inv, "interleaved")[perm])


def test_llama3_scaling_branches():
    d, theta = 24, 500000.0
    plain = P.rope_inv_freq(d, theta, None)
    sc = {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
          "original_max_position_embeddings": 32}
    got = P.rope_inv_freq(d, theta, sc)
    lam = 2 * math.pi / plain
    short, long_ = lam < 32 / 4.0, lam > 32 / 1.0
    assert short.any() and long_.any() and (~short & ~long_).any()              # all three branches
    assert torch.equal(got[short], plain[short])
    assert torch.allclose(got[long_], plain[long_] / 8.0)
    mid = ~short & ~long_
    assert torch.all(got[mid] < plain[mid]) and torch.all(got[mid] > plain[mid] / 8.0)
    assert torch.all(got[1:] < got[:-1])                                        # still monotone
    one = dict(sc, factor=1.0)
    assert torch.allclose(P.rope_inv_freq(d, theta, one), plain)
    # the engine's table builder is a different piece of code and must agree
    from rbitnet_amd.parts.position import rope_inverse_frequencies
    assert torch.allclose(rope_inverse_frequencies(d, theta, sc), got, rtol=1e-14)


def test_llama3_middle_range_is_the_one_affine_blend():
    """Between the two boundaries the scaled frequency divided by the unscaled one is an affine
    function of the frequency (the blend is linear in original / wavelength) that meets the
    branch on either side without a jump.  An affine function with both ends fixed is unique,
    so these three properties are the rule; a blend with its two weights swapped, or one linear
    in the wavelength, fails.  The frequencies lie 0.45 % apart here (head size 4096), so that
    some fall just inside either boundary."""
    d, theta = 4096, 10000.0
    orig, low, high, factor = 32, 1.0, 4.0, 8.0
    sc = {"rope_type": "llama3", "factor": factor, "low_freq_factor": low, "high_freq_factor": high,
          "original_max_position_embeddings": orig}
    plain = P.rope_inv_freq(d, theta, None)
    got = P.rope_inv_freq(d, theta, sc)
    ratio = got / plain
    lam = 2 * math.pi / plain
    step = theta ** (2.0 / d) - 1.0                                    # neighbouring wavelengths differ by this
    assert step < 0.005
    short, long_ = lam < orig / high, lam > orig / low
    mid = ~short & ~long_
    assert int(mid.sum()) > 250 and short.any() and long_.any()
    assert torch.all(ratio[short] == 1.0) and torch.allclose(ratio[long_], torch.full_like(ratio[long_], 1 / factor))
    idx = torch.nonzero(mid).flatten()
    first, last = int(idx[0]), int(idx[-1])
    # no jump at the short-wave boundary: the first middle frequency is nearly unscaled ...
    assert abs(float(ratio[first]) - 1.0) < 7.0 / 6.0 * step + 1e-12
    # ... nor at the long-wave boundary: the last one is nearly divided by the factor
    assert abs(float(ratio[last]) - 1.0 / factor) < (1 - 1 / factor) / (high - low) * step + 1e-12
    # strictly between, falling as the waves get longer
    assert torch.all(ratio[idx][1:] < ratio[idx][:-1]) and ratio[last] > 1 / factor and ratio[first] < 1.0
    # affine in the frequency: equal slopes between any neighbours
    f, r = plain[idx], ratio[idx]
    slopes = (r[1:] - r[:-1]) / (f[1:] - f[:-1])
    assert float((slopes.max() - slopes.min()) / slopes.mean().abs()) < 1e-9
    # the slope itself, from the two fixed ends: (1 - 1/factor) / (f(orig/high) - f(orig/low))
    want_slope = (1 - 1 / factor) / (2 * math.pi * high / orig - 2 * math.pi * low / orig)
    assert abs(float(slopes.mean()) / want_slope - 1.0) < 1e-9
    # the shape the large models use (head size 128, theta 5e5, original length 8192): the same
    # affine map, and the engine's table builder agrees on every frequency
    sc2 = dict(sc, original_max_position_embeddings=8192)
    p2, g2 = P.rope_inv_freq(128, 500000.0, None), P.rope_inv_freq(128, 500000.0, sc2)
    lam2 = 2 * math.pi / p2
    m2 = (lam2 >= 8192 / high) & (lam2 <= 8192 / low)
    assert int(m2.sum()) >= 6
    affine = 1 / factor + (1 - 1 / factor) * (8192 * p2[m2] / (2 * math.pi) - low) / (high - low)
    assert torch.allclose(g2[m2] / p2[m2], affine, rtol=1e-12)
    from rbitnet_amd.parts.position import rope_inverse_frequencies
    assert torch.allclose(rope_inverse_frequencies(128, 500000.0, sc2), g2, rtol=1e-14)
    assert torch.allclose(rope_inverse_frequencies(d, theta, sc), got, rtol=1e-14)


def test_half_pairing_of_a_whole_model_equals_adjacent_pairs_on_permuted_rows():
    """The two pairings of the rotation differ by a permutation of the rows of Wq and Wk inside
    every head (scores are dot products, which no common permutation changes): a model read with
    "half" and the same model with these rows permuted and read with adjacent pairs, as the
    reference rotates (model.rs:122-136), give the same logits."""
    m = P.PlainLlama.from_folder(model_folder("B"))
    assert m.style == "half"                                             # no key in config.json: names decide
    toks = [5, 6, 7, 300, 2, 9]
    d = m.head_dim
    perm = torch.stack([torch.arange(d // 2), torch.arange(d // 2) + d // 2], dim=1).reshape(-1)   # new[2i] = old[i]
    z = copy.copy(m)
    z.w = dict(m.w)
    z.style = "interleaved"
    for il in range(m.n_layer):
        for name, heads in (("q_proj", m.n_head), ("k_proj", m.n_kv)):
            key = f"model.layers.{il}.self_attn.{name}.weight"
            w = m.w[key].view(heads, d, -1)
            z.w[key] = w[:, perm, :].reshape(heads * d, -1)
    assert torch.allclose(z.logits(toks), m.logits(toks), atol=1e-12)
    z.style = "half"
    assert not torch.allclose(z.logits(toks), m.logits(toks), atol=1e-6)         # the pairing matters


def test_attention_reduces_to_library_attention():
    t, hq, hk, d = 9, 4, 2, 6
    q, k, v = torch.randn(t, hq * d, dtype=D64), torch.randn(t, hk * d, dtype=D64), torch.randn(t, hk * d, dtype=D64)
    got = P.attention(q, k, v, hq, hk)
    qq = q.view(t, hq, d).transpose(0, 1)
    kk = k.view(t, hk, d).transpose(0, 1).repeat_interleave(hq // hk, dim=0)    # q head h reads kv head h // 2
    vv = v.view(t, hk, d).transpose(0, 1).repeat_interleave(hq // hk, dim=0)
    want = F.scaled_dot_product_attention(qq, kk, vv, is_causal=True).transpose(0, 1).reshape(t, hq * d)
    assert torch.allclose(got, want, atol=1e-12)
    assert torch.allclose(got[0], v.view(t, hk, d)[0].repeat_interleave(2, dim=0).reshape(-1))   # one key: out = v
    # causal: a later token changes nothing earlier
    k2, v2 = k.clone(), v.clone()
    k2[6] += 1.0
    v2[6] -= 2.0
    assert torch.equal(P.attention(q, k2, v2, hq, hk)[:6], got[:6])
    # window: equals full attention over the last w keys
    w = 3
    gw = P.attention(q, k, v, hq, hk, window=w)
    assert torch.allclose(gw[:w], got[:w])
    last = P.attention(q[t - w:], k[t - w:], v[t - w:], hq, hk)[-1]
    assert torch.allclose(gw[-1], last)


def test_swiglu_and_one_layer_identities():
    h = torch.randn(3, 8, dtype=D64)
    wg, wu, wd = torch.randn(20, 8, dtype=D64), torch.randn(20, 8, dtype=D64), torch.randn(8, 20, dtype=D64)
    assert torch.allclose(P.swiglu(h, wg, wu, wd), F.linear(F.silu(F.linear(h, wg)) * F.linear(h, wu), wd))
    m = P.PlainLlama.from_folder(model_folder("A"))
    toks = [3, 200, 17, 5]
    base = m.logits(toks)
    # with the output projections zeroed a layer is the identity: logits = head(norm(embedding))
    z = copy.copy(m)
    z.w = dict(m.w)
    for i in range(m.n_layer):
        z.w[f"model.layers.{i}.self_attn.o_proj.weight"] = torch.zeros_like(m.w[f"model.layers.{i}.self_attn.o_proj.weight"])
        z.w[f"model.layers.{i}.mlp.down_proj.weight"] = torch.zeros_like(m.w[f"model.layers.{i}.mlp.down_proj.weight"])
    x = P.embedding(m.w["model.embed_tokens.weight"], toks)
    want = P.linear(P.rmsnorm(x, m.w["model.norm.weight"], m.eps), m.w["lm_head.weight"])
    assert torch.allclose(z.logits(toks), want)
    assert not torch.allclose(base, want)
    # logits at a position do not depend on later tokens
    assert torch.allclose(m.logits(toks + [9, 9])[:4], base)


def test_tied_head_and_shift_of_positions():
    m = P.PlainLlama.from_folder(model_folder("B"))
    toks = [5, 6, 7, 300]
    x = m.hidden(toks)
    want = P.linear(P.rmsnorm(x, m.w["model.norm.weight"], m.eps), m.w["model.embed_tokens.weight"])
    assert torch.allclose(m.logits(toks), want)
    assert "lm_head.weight" not in m.w


def test_sampling():
    logits = torch.tensor([0.1, 2.0, float("nan"), 2.0, -1.0])
    assert P.argmax_token(logits) == 1                                # NaN as -inf, lowest index among equals
    assert P.sample_token(logits, 0.0, 0.9) == 1 and P.sample_token(logits, -1.0, 0.9) == 1
    z = torch.tensor([0.0, math.log(3.0)])                            # probabilities 1/4, 3/4 at T = 1
    assert P.sample_token(z, 1.0, 0.2) == 0 and P.sample_token(z, 1.0, 0.26) == 1
    assert P.sample_token(z, 0.5, 0.09) == 0 and P.sample_token(z, 0.5, 0.11) == 1   # 1/10, 9/10 at T = 1/2
    assert P.sample_token(z, 1.0, 0.0) == 0 and P.sample_token(z, 1.0, 0.999999) == 1
    hist = [0, 0]
    for i in range(4000):
        hist[P.sample_token(z, 1.0, (i + 0.5) / 4000)] += 1
    assert abs(hist[0] / 4000 - 0.25) < 0.01


def test_forms_for_long_sequences_equal_the_loops():
    """`rope_rows`, `attention_rows` and the model's rows_at_once mode are the element-by-element
    functions written with whole-tensor operations: equal to them up to the order of float64 sums."""
    t_len, hq, hk, d = 9, 6, 2, 8
    inv = P.rope_inv_freq(d, 10000.0, None)
    x = torch.randn(t_len, hq * d, dtype=D64)
    for style in ("interleaved", "half"):
        want = torch.stack([torch.cat([P.rope(x[t, h * d:(h + 1) * d], t + 3, inv, style) for h in range(hq)])
                            for t in range(t_len)])
        assert torch.allclose(P.rope_rows(x, hq, inv, style, first_pos=3), want, atol=1e-14)
    q, k, v = x, torch.randn(t_len, hk * d, dtype=D64), torch.randn(t_len, hk * d, dtype=D64)
    for window in (None, 4):
        assert torch.allclose(P.attention_rows(q, k, v, hq, hk, window), P.attention(q, k, v, hq, hk, window),
                              atol=1e-13)
    rounded = lambda t: t.to(torch.bfloat16).to(t.dtype)
    assert torch.allclose(P.attention_rows(q, k, v, hq, hk, None, rounded),
                          P.attention(q, k, v, hq, hk, None, round_weights=rounded), atol=1e-13)
    for name in ("A", "B"):
        folder = model_folder(name)
        toks = [3, 200, 17, 5, 5, 90, 41, 7, 250, 0, 13]
        slow, fast = P.PlainLlama.from_folder(folder), P.PlainLlama.from_folder(folder, rows_at_once=True)
        assert torch.allclose(fast.logits(toks), slow.logits(toks), atol=1e-12)
        assert torch.allclose(fast.logits(toks, last=3), fast.logits(toks)[-3:], atol=1e-13)
