"""Plain, slow Llama decoder: whole sequences, no cache, one function per part.

Written from the formulas of the reference's CPU engine
(crates/bitnet-core/src/llama/model.rs and runtime.rs); every function names the
lines it follows.  It shares no code with the `rbitnet_amd` package: it reads
config.json as a plain dict, reads weights with the `safetensors` package, and
computes everything with elementary torch operations on the CPU (float64 unless
asked otherwise), so it can serve as the oracle for the engine's tests.

The three things the reference does not have (it reads GGUF, whose exporters
already applied them) are written from their definitions and marked "ours":
llama3 frequency scaling, the "half" pairing of rotary dimensions, and tied
output embeddings.
"""
from __future__ import annotations

import json
import math
import os

import torch


# --------------------------------------------------------------------------- parts

def linear(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """y[o] = sum_i W[o, i] * x[i]; W is row-major [out, in], no bias.

    model.rs:67-78 (matvec_embd_out) and model.rs:80-91 (matvec_ff_embd).
    """
    rows, n_in = x.shape
    n_out = w.shape[0]
    assert w.shape[1] == n_in
    y = torch.zeros(rows, n_out, dtype=x.dtype, device=x.device)
    for r in range(rows):
        y[r] = (w * x[r][None, :]).sum(dim=1)
    return y


def embedding(table: torch.Tensor, tokens) -> torch.Tensor:
    """x = token_embd[tok, :]; ids outside the table are an error.

    model.rs:224-232.
    """
    rows = []
    for t in tokens:
        if not 0 <= int(t) < table.shape[0]:
            raise ValueError("token id out of range")
        rows.append(table[int(t)].clone())
    return torch.stack(rows)


def rmsnorm(x: torch.Tensor, gain: torch.Tensor, eps: float) -> torch.Tensor:
    """s = mean(x^2); y_i = x_i * w_i / sqrt(s + eps); eps sits inside the root.

    model.rs:93-100.
    """
    s = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    scale = 1.0 / torch.sqrt(s + eps)
    return x * gain * scale


def softmax(s: torch.Tensor) -> torch.Tensor:
    """Subtract the maximum, exponentiate, divide by the sum (if positive).

    model.rs:102-114.
    """
    m = s.max()
    z = torch.exp(s - m)
    total = z.sum()
    if total > 0:
        z = z / total
    return z


def silu(v: torch.Tensor) -> torch.Tensor:
    """v / (1 + exp(-v)).  model.rs:116-120."""
    return v / (1.0 + torch.exp(-v))


def rope_inv_freq(head_dim: int, theta: float, scaling: dict | None) -> torch.Tensor:
    """inv_i = 1 / theta^(2i / D) for i < D/2.  model.rs:126.

    Ours (not in the reference): `scaling` with rope_type "llama3" rescales each
    frequency by its wavelength lambda = 2*pi/inv.  Short waves
    (lambda < orig/high) stay, long waves (lambda > orig/low) are divided by
    `factor`, and between the two the result is interpolated linearly in
    s = (orig/lambda - low) / (high - low).
    """
    i = torch.arange(head_dim // 2, dtype=torch.float64)
    inv = 1.0 / (float(theta) ** (2.0 * i / head_dim))
    if scaling is None:
        return inv
    kind = scaling.get("rope_type", scaling.get("type", "default"))
    if kind == "default":
        return inv
    if kind != "llama3":
        raise ValueError(f"unsupported rope_type {kind!r}")
    factor = float(scaling["factor"])
    low = float(scaling["low_freq_factor"])
    high = float(scaling["high_freq_factor"])
    orig = float(scaling["original_max_position_embeddings"])
    out = inv.clone()
    for j in range(inv.numel()):
        lam = 2.0 * math.pi / float(inv[j])
        if lam < orig / high:
            continue
        if lam > orig / low:
            out[j] = inv[j] / factor
        else:
            s = (orig / lam - low) / (high - low)
            out[j] = (1.0 - s) * inv[j] / factor + s * inv[j]
    return out


def rope(x: torch.Tensor, pos: int, inv_freq: torch.Tensor, style: str = "interleaved") -> torch.Tensor:
    """Rotate one head's vector by the angles pos * inv_i.

    "interleaved" pairs (x[2i], x[2i+1]) as the reference does, model.rs:122-136:
        x0' = x0 cos a - x1 sin a ; x1' = x0 sin a + x1 cos a.
    "half" (ours) pairs (x[i], x[i + D/2]) with the same rotation.
    """
    d = x.shape[-1]
    half = d // 2
    out = x.clone()
    for i in range(half):
        a = float(pos) * float(inv_freq[i])
        c, s = math.cos(a), math.sin(a)
        if style == "interleaved":
            i0, i1 = 2 * i, 2 * i + 1
        elif style == "half":
            i0, i1 = i, i + half
        else:
            raise ValueError(style)
        x0, x1 = x[i0], x[i1]
        out[i0] = x0 * c - x1 * s
        out[i1] = x0 * s + x1 * c
    return out


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, n_head: int, n_kv: int,
              window: int | None = None, first_pos: int = 0, round_weights=None) -> torch.Tensor:
    """Causal attention of a whole sequence, grouped heads.

    q [T, n_head*D], k and v [T, n_kv*D], already rotated.  Query head qh reads
    kv head qh // (n_head // n_kv) (model.rs:234,263); the score is the dot
    product times 1/sqrt(D), the scale applied after the sum (model.rs:260,
    269-275); keys p <= pos only (model.rs:266); softmax; weighted sum of the
    values (model.rs:278-288); heads are concatenated in head order.
    Ours: `window` keeps only the keys with pos - p < window; `round_weights`, a function,
    is applied to the exponentials exp(s - max) before they weigh the values (their sum is
    taken before it): the place where an engine that multiplies in reduced precision rounds.
    """
    t_len = q.shape[0]
    d = q.shape[1] // n_head
    n_rep = n_head // n_kv
    scale = 1.0 / math.sqrt(d)
    out = torch.zeros(t_len, n_head * d, dtype=q.dtype, device=q.device)
    for pos in range(t_len):
        lo = 0 if window is None else max(0, pos - window + 1)
        for qh in range(n_head):
            kvh = qh // n_rep
            qv = q[pos, qh * d:(qh + 1) * d]
            keys = k[lo:pos + 1, kvh * d:(kvh + 1) * d]
            scores = (keys * qv[None, :]).sum(dim=1) * scale
            if round_weights is None:
                prob = softmax(scores)
            else:
                z = torch.exp(scores - scores.max())
                prob = round_weights(z) / z.sum()
            comb = (prob[:, None] * v[lo:pos + 1, kvh * d:(kvh + 1) * d]).sum(dim=0)
            out[pos, qh * d:(qh + 1) * d] = comb
    return out


def rope_rows(x: torch.Tensor, n_heads: int, inv_freq: torch.Tensor, style: str = "interleaved",
              first_pos: int = 0) -> torch.Tensor:
    """`rope` for every row and head of x [T, n_heads * D] at once (row t at position first_pos + t):
    the same pairs, angles and signs written with whole-tensor operations, for sequences of hundreds
    of tokens at the widths of real models.  tests/test_plain.py holds it equal to `rope`."""
    t_len = x.shape[0]
    d = x.shape[1] // n_heads
    half = d // 2
    pos = torch.arange(first_pos, first_pos + t_len, dtype=torch.float64)
    a = pos[:, None] * inv_freq.to(torch.float64)[None, :]                # [T, D/2]
    c = torch.cos(a).to(device=x.device, dtype=x.dtype)[:, None, :]
    s = torch.sin(a).to(device=x.device, dtype=x.dtype)[:, None, :]
    v = x.reshape(t_len, n_heads, d)
    if style == "interleaved":
        x0, x1 = v[..., 0::2], v[..., 1::2]
    elif style == "half":
        x0, x1 = v[..., :half], v[..., half:]
    else:
        raise ValueError(style)
    y0 = x0 * c - x1 * s
    y1 = x0 * s + x1 * c
    out = torch.empty_like(v)
    if style == "interleaved":
        out[..., 0::2], out[..., 1::2] = y0, y1
    else:
        out[..., :half], out[..., half:] = y0, y1
    return out.reshape(t_len, n_heads * d)


def attention_rows(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, n_head: int, n_kv: int,
                   window: int | None = None, round_weights=None) -> torch.Tensor:
    """`attention` with one [T, T] score matrix per head in place of the loop over positions: the
    same scale, mask, maximum, sum and weighting.  tests/test_plain.py holds it equal to `attention`."""
    t_len = q.shape[0]
    d = q.shape[1] // n_head
    n_rep = n_head // n_kv
    scale = 1.0 / math.sqrt(d)
    pos = torch.arange(t_len, device=q.device)
    seen = pos[None, :] <= pos[:, None]
    if window is not None:
        seen = seen & (pos[:, None] - pos[None, :] < window)
    out = torch.zeros(t_len, n_head * d, dtype=q.dtype, device=q.device)
    for qh in range(n_head):
        kvh = qh // n_rep
        scores = (q[:, qh * d:(qh + 1) * d] @ k[:, kvh * d:(kvh + 1) * d].T) * scale
        scores = scores.masked_fill(~seen, -math.inf)
        z = torch.exp(scores - scores.max(dim=1, keepdim=True).values)
        total = z.sum(dim=1, keepdim=True)
        if round_weights is not None:
            z = round_weights(z)
        out[:, qh * d:(qh + 1) * d] = (z / total) @ v[:, kvh * d:(kvh + 1) * d]
    return out


def swiglu(h: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor) -> torch.Tensor:
    """down( silu(gate h) * (up h) ).  model.rs:297-303."""
    g = silu(linear(h, w_gate))
    u = linear(h, w_up)
    return linear(g * u, w_down)


# --------------------------------------------------------------------------- model

class PlainLlama:
    """config.json + tensors by name -> logits of whole sequences."""

    def __init__(self, config: dict, tensors: dict, dtype=torch.float64, device="cpu", round_bf16: bool = False,
                 rows_at_once: bool = False):
        """rows_at_once: rotation, attention and matrix products through `rope_rows`, `attention_rows`
        and one matrix product per call (the forms for long sequences at real widths).
        round_bf16: round to bfloat16 wherever an engine that computes in bfloat16 stores a
        value in that type (normalised rows, rotated q and k, v, the weights of the values, the
        attention output, the gated activation), everything else as before.  The distance of
        that from the exact logits is what such an engine cannot avoid; its distance from an
        engine's logits is what the engine adds."""
        c = config
        self.round_bf16 = round_bf16
        self.rows_at_once = rows_at_once
        self.dtype = dtype
        self.device = device        # where the sums run; the element-by-element rotation stays on the host
        self.n_embd = int(c["hidden_size"])
        self.n_layer = int(c["num_hidden_layers"])
        self.n_head = int(c["num_attention_heads"])
        self.n_kv = int(c.get("num_key_value_heads") or self.n_head)      # config.rs:56
        self.head_dim = int(c.get("head_dim") or self.n_embd // self.n_head)  # config.rs:62
        self.n_ff = int(c["intermediate_size"])
        self.n_vocab = int(c["vocab_size"])
        self.theta = float(c.get("rope_theta", 10000.0))                   # config.rs:94-97
        self.eps = float(c.get("rms_norm_eps", 1e-5))                      # config.rs:99-102
        self.scaling = c.get("rope_scaling")
        # without the key: "half", the layout of weights stored under these names (this class
        # reads `model.layers.N...` names only); the reference's adjacent pairs fit GGUF files,
        # whose q and k rows were permuted for them when they were exported
        self.style = c.get("rope_style") or "half"
        self.tied = bool(c.get("tie_word_embeddings", False))
        self.window = c.get("sliding_window")
        self.inv_freq = rope_inv_freq(self.head_dim, self.theta, self.scaling)
        self.w = {k: v.to(device=device, dtype=dtype) for k, v in tensors.items()}

    @classmethod
    def from_folder(cls, folder: str, dtype=torch.float64, device="cpu", round_bf16: bool = False,
                    rows_at_once: bool = False) -> "PlainLlama":
        from safetensors.torch import load_file
        with open(os.path.join(folder, "config.json")) as f:
            config = json.load(f)
        tensors = load_file(os.path.join(folder, "model.safetensors"))
        return cls(config, tensors, dtype, device, round_bf16, rows_at_once)

    def _r(self, t: torch.Tensor) -> torch.Tensor:
        return t.to(torch.bfloat16).to(t.dtype) if self.round_bf16 else t

    def layer(self, x: torch.Tensor, il: int) -> torch.Tensor:
        """One block: norm, q/k/v, rotate q and k, attention, output projection
        and residual, norm, feed-forward and residual.  model.rs:236-307."""
        p = f"model.layers.{il}."
        w = self.w
        d = self.head_dim
        lin = self._linear
        h = self._r(rmsnorm(x, w[p + "input_layernorm.weight"], self.eps))
        q = lin(h, w[p + "self_attn.q_proj.weight"])
        k = lin(h, w[p + "self_attn.k_proj.weight"])
        v = lin(h, w[p + "self_attn.v_proj.weight"])
        if self.rows_at_once:
            q = rope_rows(q, self.n_head, self.inv_freq, self.style)
            k = rope_rows(k, self.n_kv, self.inv_freq, self.style)
        else:
            q, k = q.cpu(), k.cpu()
            for pos in range(x.shape[0]):
                for hh in range(self.n_head):
                    q[pos, hh * d:(hh + 1) * d] = rope(q[pos, hh * d:(hh + 1) * d], pos, self.inv_freq, self.style)
                for hh in range(self.n_kv):
                    k[pos, hh * d:(hh + 1) * d] = rope(k[pos, hh * d:(hh + 1) * d], pos, self.inv_freq, self.style)
        q, k, v = self._r(q.to(x.device)), self._r(k.to(x.device)), self._r(v)
        attend = attention_rows if self.rows_at_once else attention
        a = self._r(attend(q, k, v, self.n_head, self.n_kv, self.window,
                           round_weights=self._r if self.round_bf16 else None))
        x = x + lin(a, w[p + "self_attn.o_proj.weight"])
        h2 = self._r(rmsnorm(x, w[p + "post_attention_layernorm.weight"], self.eps))
        if self.round_bf16 or self.rows_at_once:
            t = self._r(silu(lin(h2, w[p + "mlp.gate_proj.weight"])) * lin(h2, w[p + "mlp.up_proj.weight"]))
            return x + lin(t, w[p + "mlp.down_proj.weight"])
        x = x + swiglu(h2, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                       w[p + "mlp.down_proj.weight"])
        return x

    def _linear(self, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
        return x @ w.T if self.rows_at_once else linear(x, w)

    def hidden(self, tokens) -> torch.Tensor:
        x = embedding(self.w["model.embed_tokens.weight"], tokens)
        for il in range(self.n_layer):
            x = self.layer(x, il)
        return x

    def logits(self, tokens, last: int | None = None) -> torch.Tensor:
        """Logits [T, V] at every position of one sequence (`last`: at its last that many
        positions only).  model.rs:229-315."""
        x = self.hidden(tokens)
        if last is not None:
            x = x[-last:]
        xn = self._r(rmsnorm(x, self.w["model.norm.weight"], self.eps))
        head = self.w["model.embed_tokens.weight"] if self.tied else self.w["lm_head.weight"]
        return self._linear(xn, head)


# --------------------------------------------------------------------------- sampling

def argmax_token(logits: torch.Tensor) -> int:
    """Greatest logit, NaN counted as -inf (runtime.rs:82-93); among equal
    maxima the lowest index (the engine's documented rule; the reference's
    iterator keeps the last)."""
    best, best_v = 0, -math.inf
    for i, val in enumerate(logits.tolist()):
        val = -math.inf if val != val else val
        if val > best_v:
            best, best_v = i, val
    return best


def sample_token(logits: torch.Tensor, temperature: float, u: float) -> int:
    """temperature <= 0 -> argmax; else z = logits / T, e = exp(z - max z),
    r = u * sum(e), first index whose running sum reaches r, else the last
    index.  runtime.rs:81-107 with the uniform number u given by the caller."""
    if temperature <= 0.0:
        return argmax_token(logits)
    z = logits.to(torch.float64) / temperature
    e = torch.exp(z - z.max())
    r = u * float(e.sum())
    c = 0.0
    for i, val in enumerate(e.tolist()):
        c += val
        if c >= r:
            return i
    return len(e) - 1


def greedy_generate(model: PlainLlama, prompt, max_tokens: int, stop=()) -> list:
    """Greedy loop of runtime.rs:61-73 with whole-sequence recomputation: sample,
    stop before emitting a stop token, append, run again."""
    seq = list(prompt)
    out = []
    for _ in range(max_tokens):
        nxt = argmax_token(model.logits(seq)[-1])
        if nxt in stop:
            break
        out.append(nxt)
        seq.append(nxt)
    return out
