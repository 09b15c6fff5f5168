"""The plain C++ twins of the kernels (rbitnet_amd/csrc/plain.cpp) on the CPU: their self-test
under the address and undefined-behaviour sanitizers, each twin against the function of the
plain implementation that states the same formula, and a whole tiny model stepped through the
twins alone (a paged cache, prompts and single tokens) against the plain implementation's logits.
No GPU."""
import subprocess

import pytest
import torch

import plain_llama as P
from helpers import CONFIGS, model_folder, tokens_for
from rbitnet_amd.csrc import build
from rbitnet_amd.csrc.plain import plain_kernels

D64 = torch.float64
I32 = torch.int32


@pytest.fixture(scope="module")
def twin():
    return plain_kernels()


def test_self_test_under_the_sanitizers():
    exe = build.build_plain_selftest()
    run = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, run.stdout + run.stderr
    assert "plain twins ok" in run.stdout


def test_products_and_reference_vectors(twin):
    # crates/bitnet-core/src/kernels.rs:35-40 and tests/golden_kernels.rs:12-18
    c = torch.empty(1, 2)
    twin.gemm_generic(torch.tensor([[2., 3.]]), torch.tensor([[1., 0.], [-1., 1.]]), c)
    assert c.tolist() == [[2., 1.]]
    w = torch.tensor([[1., -1, 0, 1], [0, 1, 1, -1], [1, 0, -1, 0]])
    c = torch.empty(1, 3)
    twin.gemm_generic(torch.tensor([[0.5, -0.25, 2.0, 1.0]]), w, c)
    assert c.tolist() == [[1.75, 0.75, -1.5]]
    g = torch.Generator().manual_seed(0)
    x, w = torch.randn(5, 96, generator=g), torch.randn(40, 96, generator=g)
    c = torch.empty(5, 40)
    twin.gemm_generic(x, w, c)
    assert torch.allclose(c.double(), P.linear(x.double(), w.double()), atol=1e-5)
    xb, wb = x.bfloat16(), w.bfloat16()
    c2 = torch.empty(5, 40)
    twin.gemm_bf16(xb, wb, c2)
    assert torch.allclose(c2.double(), P.linear(xb.double(), wb.double()), atol=1e-5)


def test_embedding_norm_and_gate(twin):
    g = torch.Generator().manual_seed(1)
    table = torch.randn(11, 7, generator=g)
    out = torch.empty(3, 7)
    twin.embed_gather(table, torch.tensor([10, 0, 3], dtype=I32), out)
    assert torch.equal(out, P.embedding(table, [10, 0, 3]))
    x, delta, gain = torch.randn(4, 33, generator=g), torch.randn(4, 33, generator=g), torch.randn(33, generator=g)
    for eps in (1e-5, 1e-2):
        xs = x.clone()
        out = torch.empty(4, 33)
        twin.add_rmsnorm(xs, delta, gain, eps, None, out)
        assert torch.equal(xs, x + delta)
        assert torch.allclose(out.double(), P.rmsnorm((x + delta).double(), gain.double(), eps), atol=1e-6)
    gu = torch.randn(3, 2 * 20, generator=g) * 3
    t = torch.empty(3, 20)
    twin.swiglu(gu, t)
    assert torch.allclose(t.double(), P.silu(gu[:, :20].double()) * gu[:, 20:].double(), atol=1e-6)


@pytest.mark.parametrize("style", ["interleaved", "half"])
def test_rotation_cache_write_and_attention(twin, style):
    """One sequence of 70 tokens (two pages, stored out of order) through rope_kv_write and the
    attention twin, against P.rope and P.attention on the whole sequence; then its last token
    through the fused decode form."""
    hq, hk, d, t_len = 4, 2, 8, 70
    g = torch.Generator().manual_seed(2)
    qkv = torch.randn(t_len, (hq + 2 * hk) * d, generator=g)
    inv = P.rope_inv_freq(d, 10000.0, None)
    angles = torch.arange(t_len, dtype=D64)[:, None] * inv[None, :]
    cos, sin = torch.cos(angles).float().contiguous(), torch.sin(angles).float().contiguous()
    pos = torch.arange(t_len, dtype=I32)
    seq = torch.zeros(t_len, dtype=I32)
    bt = torch.tensor([[2, 0]], dtype=I32)
    kp, vp = torch.full((3, hk, 64, d), float("nan")), torch.full((3, hk, 64, d), float("nan"))
    q = torch.empty(t_len, hq, d)
    twin.rope_kv_write(qkv, cos, sin, 0 if style == "interleaved" else 1, q, kp, vp, pos, seq, bt, hq, hk, d)
    out = torch.empty(t_len, hq * d)
    twin.attention_generic(q, kp, vp, out, pos, seq, bt, hq, hk, d, d ** -0.5, 0)
    qd = qkv.double()
    q_want = P.rope_rows(qd[:, :hq * d], hq, inv, style)
    k_want = P.rope_rows(qd[:, hq * d:(hq + hk) * d], hk, inv, style)
    one = torch.cat([P.rope(qd[5, h * d:(h + 1) * d], 5, inv, style) for h in range(hq)])      # and the element-wise form
    assert torch.allclose(q.reshape(t_len, -1)[5].double(), one, atol=1e-6)
    want = P.attention(q_want, k_want, qd[:, (hq + hk) * d:], hq, hk)
    assert torch.allclose(q.reshape(t_len, -1).double(), q_want, atol=1e-6)
    assert torch.allclose(out.double(), want, atol=1e-5)
    # a window of 9 keys
    twin.attention_generic(q, kp, vp, out, pos, seq, bt, hq, hk, d, d ** -0.5, 9)
    assert torch.allclose(out.double(), P.attention(q_want, k_want, qd[:, (hq + hk) * d:], hq, hk, window=9), atol=1e-5)
    # bfloat16 storage, the last token alone through the fused decode form
    kb, vb = kp.bfloat16(), vp.bfloat16()
    ob = torch.empty(1, hq * d, dtype=torch.bfloat16)
    twin.attention_decode_fused_bf16(qkv[-1:].contiguous(), cos, sin, 0 if style == "interleaved" else 1, kb, vb, ob,
                                     pos[-1:].contiguous(), bt, hq, hk, d, d ** -0.5, 0)
    assert torch.allclose(ob.double(), want[-1:], atol=3e-2)


def test_choice_of_the_next_token(twin):
    g = torch.Generator().manual_seed(3)
    logits = torch.randn(6, 300, generator=g) * 3
    logits[0, 17] = logits[0].max() + 1
    logits[0, 200] = logits[0, 17]                     # equal maxima: the lowest index
    logits[0, 5] = float("nan")                        # a row that is only ever taken the maximum of
    tok = torch.empty(6, dtype=I32)
    twin.sample(logits, None, None, tok)
    assert tok.tolist() == [P.argmax_token(row) for row in logits]
    temps = torch.tensor([0.0, 0.7, 1.3, 0.2, 2.0, 1.0])
    us = torch.tensor([0.3, 0.0, 0.999, 0.5, 0.25, 0.75])
    twin.sample(logits, temps, us, tok)
    assert tok.tolist() == [P.sample_token(row, float(t), float(u)) for row, t, u in zip(logits, temps, us)]


class TwinModel:
    """A Llama decoder stepped through the twins alone, the way the engine steps it through the
    kernels: packed tokens, q/k/v rows in one matrix, a cache in pages, the residual sum done
    by the norm that follows."""

    def __init__(self, twin, folder, dtype):
        import json
        import os
        from safetensors.torch import load_file
        with open(os.path.join(folder, "config.json")) as f:
            c = json.load(f)
        self.twin, self.dtype = twin, dtype
        self.w = {k: v.to(dtype if v.dim() == 2 else torch.float32) for k, v in
                  load_file(os.path.join(folder, "model.safetensors")).items()}
        self.e, self.layers = c["hidden_size"], c["num_hidden_layers"]
        self.hq, self.hk = c["num_attention_heads"], c["num_key_value_heads"]
        self.d = c.get("head_dim") or self.e // self.hq
        self.ff, self.eps, self.tied = c["intermediate_size"], c["rms_norm_eps"], c.get("tie_word_embeddings", False)
        self.style = 0 if c.get("rope_style") == "interleaved" else 1
        inv = P.rope_inv_freq(self.d, c.get("rope_theta", 10000.0), c.get("rope_scaling"))
        angles = torch.arange(c["max_position_embeddings"], dtype=D64)[:, None] * inv[None, :]
        self.cos, self.sin = torch.cos(angles).float().contiguous(), torch.sin(angles).float().contiguous()
        self.qkv = []
        for i in range(self.layers):
            p = f"model.layers.{i}.self_attn."
            packed = torch.empty(((self.hq + 2 * self.hk) * self.d, self.e), dtype=dtype)
            row = 0
            for name in ("q", "k", "v"):
                t = self.w[p + name + "_proj.weight"].contiguous()
                twin.place_rows(t, packed, row0=row)
                row += t.shape[0]
            self.qkv.append(packed)
        n_pages = 8
        self.k = [torch.full((n_pages, self.hk, 64, self.d), float("nan"), dtype=dtype) for _ in range(self.layers)]
        self.v = [torch.full((n_pages, self.hk, 64, self.d), float("nan"), dtype=dtype) for _ in range(self.layers)]

    def _linear(self, x, w):
        out = torch.empty(x.shape[0], w.shape[0])
        (self.twin.gemm_generic if self.dtype == torch.float32 else self.twin.gemm_bf16)(x, w.contiguous(), out)
        return out

    def step(self, tokens_per_seq, past, tables):
        """tokens_per_seq[b]: the tokens sequence b brings on top of past[b]; tables[b]: its pages.
        Returns float32 logits of every token, packed."""
        tw, e = self.twin, self.e
        ids = torch.tensor([t for toks in tokens_per_seq for t in toks], dtype=I32)
        n = ids.numel()
        pos = torch.tensor([past[b] + i for b, toks in enumerate(tokens_per_seq) for i in range(len(toks))], dtype=I32)
        seq = torch.tensor([b for b, toks in enumerate(tokens_per_seq) for _ in toks], dtype=I32)
        width = max(len(t) for t in tables)
        bt = torch.tensor([list(t) + [0] * (width - len(t)) for t in tables], dtype=I32)
        x = torch.empty(n, e)
        tw.embed_gather(self.w["model.embed_tokens.weight"], ids, x)
        delta = None
        for i in range(self.layers):
            p = f"model.layers.{i}."
            h = torch.empty(n, e, dtype=self.dtype)
            tw.add_rmsnorm(x, delta, self.w[p + "input_layernorm.weight"], self.eps, None, h)
            qkv = self._linear(h, self.qkv[i])
            q = torch.empty(n, self.hq, self.d, dtype=self.dtype)
            tw.rope_kv_write(qkv, self.cos, self.sin, self.style, q, self.k[i], self.v[i], pos, seq, bt, self.hq, self.hk, self.d)
            a = torch.empty(n, self.hq * self.d, dtype=self.dtype)
            tw.attention_generic(q, self.k[i], self.v[i], a, pos, seq, bt, self.hq, self.hk, self.d, self.d ** -0.5, 0)
            delta = self._linear(a, self.w[p + "self_attn.o_proj.weight"])
            h2 = torch.empty(n, e, dtype=self.dtype)
            tw.add_rmsnorm(x, delta, self.w[p + "post_attention_layernorm.weight"], self.eps, None, h2)
            gu = self._linear(h2, torch.cat([self.w[p + "mlp.gate_proj.weight"], self.w[p + "mlp.up_proj.weight"]]))
            t = torch.empty(n, self.ff, dtype=self.dtype)
            tw.swiglu(gu, t)
            delta = self._linear(t, self.w[p + "mlp.down_proj.weight"])
        xn = torch.empty(n, e, dtype=self.dtype)
        tw.add_rmsnorm(x, delta, self.w["model.norm.weight"], self.eps, None, xn)
        return self._linear(xn, self.w["model.embed_tokens.weight" if self.tied else "lm_head.weight"])


@pytest.mark.parametrize("name", ["A", "B"])
def test_a_model_stepped_through_the_twins(twin, name):
    """Two sequences of unequal lengths: the prompts in one step, then one token each, the cache
    pages out of order.  float32 twins equal the plain implementation; bfloat16 twins stay within
    the bound the engine is held to."""
    lengths = [70, 9]
    reqs = [tokens_for(name, n, 90 + i) for i, n in enumerate(lengths)]
    want = [P.PlainLlama.from_folder(model_folder(name), rows_at_once=True).logits(r) for r in reqs]
    for dtype, tol in ((torch.float32, 2e-5), (torch.bfloat16, 3e-2)):
        model = TwinModel(twin, model_folder(name), dtype)
        tables = [[5, 1], [3]]
        cut = [n - 3 for n in lengths]
        logits = model.step([r[:c] for r, c in zip(reqs, cut)], [0, 0], tables)
        got = [[logits[:cut[0]]], [logits[cut[0]:]]]
        for j in range(3):
            step = model.step([[r[c + j]] for r, c in zip(reqs, cut)], [c + j for c in cut], tables)
            got[0].append(step[0:1])
            got[1].append(step[1:2])
        for g, w in zip(got, want):
            err = float((torch.cat(g).double() - w).abs().max() / w.abs().max())
            assert err < tol, (name, dtype, err)
    assert CONFIGS[name][0]["num_hidden_layers"] == model.layers
