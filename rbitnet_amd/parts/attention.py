"""The attention mixer: grouped-query causal attention over the paged cache.

Reference, one token (crates/bitnet-core/src/llama/model.rs:238-294): q = Wq h, k = Wk h,
v = Wv h; rotate every q head and k head; store k (rotated) and v at the token's
position; for q head qh read kv head qh / (Hq / Hk); scores (q . k) * scale over the
keys up to the token's own position; softmax; weighted sum of v; heads concatenated;
out = Wo attn.  Here the same runs for all tokens of a step at once: keys and values
of the whole step are written to the cache first, then every token attends to the
cache up to its own position, so a step may bring any number of tokens per sequence
on top of any past.

Parameters: num_heads, num_kv_heads, head_dim, scale, window (None: all keys; n: the
last n keys including the token's own), position (a PartSpec), cache_from (None, or the
index of the layer whose cache this layer reads instead of keeping one), names (tensor
names of the four matrices relative to the layer's prefix).

Interface of a mixer:
  tensor_specs() / load(tensors)
  cache_request() -> CacheRequest or None
  forward(h [T, E] compute dtype, ctx, view) -> float32 [T, E]
Two things a mixer may say of itself (this one does both):
  adds_to_stream: forward also takes stream=x (float32 [T, E], the residual stream) and
  next_norm (the norm that follows) and may add its result to the stream itself; it then returns
  None, or the GainedRows that its last product left for next_norm;
  takes_gained_rows: h may be such GainedRows instead of a tensor.
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..errors import ConfigError
from .base import BuildEnv, CacheRequest, Part, TensorSpec, build_part, register_mixer
from .linear import linear, linear_or_terms, linear_to_stream, pack_rows

DEFAULT_NAMES = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight"}
_MATRIX_CORE_HEAD_DIMS = (64, 128)
_DECODE_GROUPS = tuple(range(1, 17))    # query heads per kv head the decode kernels take


class Attention(Part):
    graph_safe = True
    plan_safe = True
    takes_gained_rows = True
    adds_to_stream = True

    def __init__(self, params: Dict, env: BuildEnv):
        self.env = env
        self.n_heads = int(params["num_heads"])
        self.n_kv = int(params["num_kv_heads"])
        self.head_dim = int(params["head_dim"])
        if self.n_heads <= 0 or self.n_kv <= 0 or self.n_heads % self.n_kv != 0:
            raise ConfigError(f"attention: {self.n_heads} heads cannot share {self.n_kv} kv heads")
        if self.head_dim <= 0 or self.head_dim % 2 != 0 or self.head_dim > 256:
            raise ConfigError(f"attention: head_dim {self.head_dim} not supported (even, at most 256)")
        self.scale = float(params.get("scale") or self.head_dim ** -0.5)
        self.window = params.get("window")
        if self.window is not None and int(self.window) <= 0:
            raise ConfigError("attention: window must be positive")
        self.cache_from = params.get("cache_from")
        self.names = dict(DEFAULT_NAMES, **(params.get("names") or {}))
        self.position = build_part("position", params["position"], env)
        self.plan_safe = bool(getattr(self.position, "plan_safe", False))
        self.hidden = env.hidden_size
        self.w_qkv: Optional[torch.Tensor] = None
        self.w_q: Optional[torch.Tensor] = None
        self.w_o: Optional[torch.Tensor] = None

    # ------------------------------------------------------------------ tensors
    def tensor_specs(self) -> Dict[str, TensorSpec]:
        qd, kd = self.n_heads * self.head_dim, self.n_kv * self.head_dim
        specs = {self.names["q"]: TensorSpec((qd, self.hidden)), self.names["o"]: TensorSpec((self.hidden, qd))}
        if self.cache_from is None:
            specs[self.names["k"]] = TensorSpec((kd, self.hidden))
            specs[self.names["v"]] = TensorSpec((kd, self.hidden))
        return specs

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        # q, k and v rows in one matrix: one product per step instead of three
        lib, allowed = self.env.lib, not getattr(self.env, "generic_only", False)
        names = ("q", "k", "v") if self.cache_from is None else ("q",)
        pieces, row = [], 0
        for n in names:
            t = tensors[self.names[n]]
            pieces.append((t, row, None, None))
            row += t.shape[0]
        first = pieces[0][0]
        self.w_qkv = pack_rows(lib, pieces, row, self.hidden, first.dtype, first.device, allowed)
        o = tensors[self.names["o"]]
        self.w_o = pack_rows(lib, [(o, 0, None, None)], o.shape[0], o.shape[1], o.dtype, o.device, allowed)

    def cache_request(self) -> Optional[CacheRequest]:
        if self.cache_from is not None:
            return None
        return CacheRequest("kv", heads=self.n_kv, head_dim=self.head_dim,
                            window=None if self.window is None else int(self.window))

    # ------------------------------------------------------------------ forward
    def forward(self, h, ctx, view, stream: Optional[torch.Tensor] = None, next_norm=None):
        lib = self.env.lib
        t = h.shape[0]
        hq, hk, d = self.n_heads, self.n_kv, self.head_dim
        owns = self.cache_from is None
        # q, k and v of the step; as the terms of the product where the position part reads such
        if getattr(self.position, "takes_terms", False):
            qkv = linear_or_terms(lib, h, self.w_qkv)
        else:
            qkv = linear(lib, h, self.w_qkv, torch.float32)
        bt = view.block_table
        attn = torch.empty((t, hq * d), dtype=self.env.dtype, device=h.device)
        window = int(self.window) if self.window is not None else 0
        fast = (self.env.dtype == torch.bfloat16 and d in _MATRIX_CORE_HEAD_DIMS
                and not getattr(self.env, "generic_only", False))
        decode = fast and ctx.max_q_len == 1 and (hq // hk) in _DECODE_GROUPS
        tables = getattr(self.position, "rotation_tables", None)
        if decode and owns and tables is not None:
            # one kernel: rotation, cache write, attention over the pages
            cos, sin, style = tables()
            n_splits, workspace = ctx.decode_workspace(hq, d, hk)
            lib.attention_decode_fused_bf16(qkv, cos, sin, style, view.k_pages, view.v_pages, attn, ctx.tok_pos, bt,
                                            hq, hk, d, self.scale, window, n_splits, workspace)
            return linear_to_stream(lib, attn, self.w_o, stream, next_norm)
        q = torch.empty((t, hq, d), dtype=self.env.dtype, device=h.device)
        if owns:
            self.position.encode_and_store(qkv, q, view.k_pages, view.v_pages, ctx, bt, hq, hk, d)
        else:
            self.position.encode_and_store(qkv, q, None, None, ctx, bt, hq, 0, d)
        if decode:
            n_splits, workspace = ctx.decode_workspace(hq, d, hk)
            lib.attention_decode_bf16(q, view.k_pages, view.v_pages, attn, ctx.tok_pos, bt, hq, hk, d,
                                      self.scale, window, n_splits, workspace)
        elif fast:
            lib.attention_prefill_bf16(q, view.k_pages, view.v_pages, attn, ctx.cu_seqlens, ctx.past_len, bt,
                                       ctx.n_seqs, ctx.max_q_len, hq, hk, d, self.scale, window)
        else:
            lib.attention_generic(q, view.k_pages, view.v_pages, attn, ctx.tok_pos, ctx.tok_seq, bt, hq, hk, d,
                                  self.scale, window)
        return linear_to_stream(lib, attn, self.w_o, stream, next_norm)


register_mixer("attention", Attention)
