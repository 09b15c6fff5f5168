"""ctypes binding of the plain C++ twins (plain.h): the methods of `lib.Kernels` under the same
names with the same arguments, on CPU tensors.  No GPU and no HIP: the library is built by the
host compiler at first use.  The twins are the kernels' oracle in the tests; nothing on the
product path calls them."""
from __future__ import annotations

import ctypes
import threading
from typing import Optional

import torch

from ..errors import KernelError
from . import build as _build

_P, _I, _F, _LL = ctypes.c_void_p, ctypes.c_int, ctypes.c_float, ctypes.c_longlong


def _code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return 0
    if dtype == torch.bfloat16:
        return 1
    raise KernelError(f"the twins take float32 or bfloat16 storage, not {dtype}")


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    if t is None:
        return None
    if t.is_cuda or not t.is_contiguous():
        raise KernelError("the twins take contiguous CPU tensors")
    return t.data_ptr()


def _terms(qkv: torch.Tensor):
    if qkv.dim() == 3:
        return qkv.shape[1], qkv.shape[0], qkv.shape[1] * qkv.shape[2]
    return qkv.shape[0], 1, 0


class PlainKernels:
    def __init__(self, path: Optional[str] = None):
        self.path = path or _build.build_plain()
        L = self._lib = ctypes.CDLL(self.path)
        L.rbp_last_error.restype = ctypes.c_char_p
        sig = {
            "rbp_embed_gather": [_P, _I, _P, _P, _I, _I, _P],
            "rbp_add_rmsnorm": [_P, _P, _I, _LL, _P, _F, _P, _I, _I, _P, _I, _P],
            "rbp_rope_kv_write": [_P, _I, _LL, _P, _P, _I, _P, _P, _P, _I, _P, _P, _P, _I, _I, _I, _I, _I, _P],
            "rbp_swiglu": [_P, _P, _I, _I, _I, _P],
            "rbp_gemm_generic": [_P, _P, _I, _P, _I, _I, _I, _I, _I, _P],
            "rbp_gemm_bf16": [_P, _P, _I, _P, _I, _I, _I, _I, _I, _P, _P],
            "rbp_gemm_bf16_few": [_P, _P, _F, _P, _P, _I, _P, _I, _I, _P, _P, _P, _I, _I, _I, _P],
            "rbp_attention_generic": [_P, _P, _P, _P, _I, _P, _P, _P, _I, _I, _I, _I, _I, _F, _I, _P],
            "rbp_attention_prefill_bf16": [_P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _F, _I, _P],
            "rbp_attention_decode_bf16": [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _F, _I, _I, _P, _P],
            "rbp_attention_decode_fused_bf16": [_P, _I, _LL, _P, _P, _I, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _F, _I, _I,
                                                _P, _P],
            "rbp_sample": [_P, _I, _I, _P, _P, _P, _P, _P],
            "rbp_place_rows": [_P, _I, _P, _I, _I] + [_LL] * 6 + [_P],
        }
        for name, args in sig.items():
            fn = getattr(L, name)
            fn.argtypes, fn.restype = args, _I
        self.page_size = int(L.rbp_page_size())

    def _ok(self, rc: int) -> None:
        if rc != 0:
            raise KernelError(self._lib.rbp_last_error().decode("utf-8", "replace"))

    def embed_gather(self, table, ids, out) -> None:
        n, width = out.shape
        self._ok(self._lib.rbp_embed_gather(_ptr(table), _code(table.dtype), _ptr(ids), _ptr(out), n, width, None))

    def add_rmsnorm(self, x, delta, gain, eps, rows, out) -> None:
        n_rows, width = out.shape
        n_terms, stride = (delta.shape[0], x.numel()) if delta is not None and delta.dim() == 3 else (1, 0)
        self._ok(self._lib.rbp_add_rmsnorm(_ptr(x), _ptr(delta), n_terms, stride, _ptr(gain), float(eps), _ptr(rows),
                                           n_rows, width, _ptr(out), _code(out.dtype), None))

    def rope_kv_write(self, qkv, cos, sin, style, q_out, k_pages, v_pages, tok_pos, tok_seq, block_table, n_heads, n_kv,
                      head_dim) -> None:
        n, n_terms, stride = _terms(qkv)
        self._ok(self._lib.rbp_rope_kv_write(_ptr(qkv), n_terms, stride, _ptr(cos), _ptr(sin), int(style), _ptr(q_out),
                                             _ptr(k_pages), _ptr(v_pages), _code(q_out.dtype), _ptr(tok_pos),
                                             _ptr(tok_seq), _ptr(block_table), block_table.shape[1], n, n_heads, n_kv,
                                             head_dim, None))

    def swiglu(self, gu, out) -> None:
        n, ff = out.shape
        self._ok(self._lib.rbp_swiglu(_ptr(gu), _ptr(out), _code(out.dtype), n, ff, None))

    def gemm_generic(self, a, w, c, w_frag: bool = False) -> None:
        m, k = a.shape
        self._ok(self._lib.rbp_gemm_generic(_ptr(a), _ptr(w), int(bool(w_frag)), _ptr(c), _code(a.dtype), _code(c.dtype),
                                            m, w.shape[0], k, None))

    def gemm_bf16(self, a, w, c, epilogue: int = 0, w_frag: bool = False) -> None:
        m, k = a.shape
        self._ok(self._lib.rbp_gemm_bf16(_ptr(a), _ptr(w), int(bool(w_frag)), _ptr(c), _code(c.dtype), int(epilogue), m,
                                         w.shape[0], k, None, None))

    def gemm_bf16_few(self, a, w, c, epilogue: int = 0, squares=None, eps: float = 0.0, rows=None, gain=None,
                      gained=None, squares_out=None, w_frag: bool = False) -> None:
        n, k = w.shape
        m = a.shape[0] if rows is None else rows.shape[0]
        self._ok(self._lib.rbp_gemm_bf16_few(_ptr(a), _ptr(squares), float(eps), _ptr(rows), _ptr(w), int(bool(w_frag)),
                                             _ptr(c), _code(c.dtype), int(epilogue), _ptr(gain), _ptr(gained),
                                             _ptr(squares_out), m, n, k, None))

    def attention_generic(self, q, k_pages, v_pages, out, tok_pos, tok_seq, block_table, n_heads, n_kv, head_dim, scale,
                          window) -> None:
        self._ok(self._lib.rbp_attention_generic(_ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(out), _code(q.dtype),
                                                 _ptr(tok_pos), _ptr(tok_seq), _ptr(block_table), block_table.shape[1],
                                                 q.shape[0], n_heads, n_kv, head_dim, float(scale), int(window or 0),
                                                 None))

    def attention_prefill_bf16(self, q, k_pages, v_pages, out, cu_seqlens, past_len, block_table, n_seqs, max_q_len,
                               n_heads, n_kv, head_dim, scale, window) -> None:
        self._ok(self._lib.rbp_attention_prefill_bf16(_ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(out), _ptr(cu_seqlens),
                                                      _ptr(past_len), _ptr(block_table), block_table.shape[1], n_seqs,
                                                      int(max_q_len), n_heads, n_kv, head_dim, float(scale),
                                                      int(window or 0), None))

    def attention_decode_bf16(self, q, k_pages, v_pages, out, tok_pos, block_table, n_heads, n_kv, head_dim, scale,
                              window, n_splits=1, workspace=None) -> None:
        self._ok(self._lib.rbp_attention_decode_bf16(_ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(out), _ptr(tok_pos),
                                                     _ptr(block_table), block_table.shape[1], q.shape[0], n_heads, n_kv,
                                                     head_dim, float(scale), int(window or 0), int(n_splits), None, None))

    def attention_decode_fused_bf16(self, qkv, cos, sin, style, k_pages, v_pages, out, tok_pos, block_table, n_heads,
                                    n_kv, head_dim, scale, window, n_splits=1, workspace=None) -> None:
        n, n_terms, stride = _terms(qkv)
        self._ok(self._lib.rbp_attention_decode_fused_bf16(
            _ptr(qkv), n_terms, stride, _ptr(cos), _ptr(sin), int(style), _ptr(k_pages), _ptr(v_pages), _ptr(out),
            _ptr(tok_pos), _ptr(block_table), block_table.shape[1], n, n_heads, n_kv, head_dim, float(scale),
            int(window or 0), int(n_splits), None, None))

    def sample(self, logits, temperature, u, tokens, workspace=None) -> None:
        n, vocab = logits.shape
        self._ok(self._lib.rbp_sample(_ptr(logits), n, vocab, _ptr(temperature), _ptr(u), _ptr(tokens), None, None))

    def place_rows(self, src, dst, row0: int = 0, block: Optional[int] = None, period: Optional[int] = None,
                   frag: bool = False) -> None:
        n = src.shape[0]
        block = max(1, n) if block is None else int(block)
        period = block if period is None else int(period)
        self._ok(self._lib.rbp_place_rows(_ptr(src), _code(src.dtype), _ptr(dst), _code(dst.dtype), int(bool(frag)), n,
                                          src.shape[1], dst.shape[0], int(row0), block, period, None))


_lock = threading.Lock()
_instance: Optional[PlainKernels] = None


def plain_kernels() -> PlainKernels:
    """The process-wide library of twins, built at first use."""
    global _instance
    with _lock:
        if _instance is None:
            _instance = PlainKernels()
        return _instance
