"""ctypes binding of librbitnet_hip.so: torch tensors in, kernels launched on torch's
current HIP stream.  There is no fallback: without a GPU and the built library every
call fails with a KernelError."""
from __future__ import annotations

import atexit
import ctypes
import os
import sys
import threading
from typing import Dict, List, Optional, Tuple

import torch

from ..errors import KernelError
from . import build as _build

_RAW_STREAM = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_F32, _BF16 = 0, 1
_P = ctypes.c_void_p
_I = ctypes.c_int
_F = ctypes.c_float


def dtype_code(dtype: torch.dtype) -> int:
    if dtype == torch.float32:
        return _F32
    if dtype == torch.bfloat16:
        return _BF16
    raise KernelError(f"the kernels take float32 or bfloat16 storage, not {dtype}")


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    if t is None:
        return None
    return t.data_ptr()


def _check(t: torch.Tensor, name: str, dtype=None, shape=None) -> None:
    if not t.is_cuda:
        raise KernelError(f"{name} must be on the GPU")
    if not t.is_contiguous():
        raise KernelError(f"{name} must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name} must be {dtype}, found {t.dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise KernelError(f"{name} must have shape {tuple(shape)}, found {tuple(t.shape)}")


def _terms(qkv: torch.Tensor, width: int):
    """qkv [T, width], or [P, T, width]: P terms to be added up in their order.  -> (T, P, stride)"""
    if qkv.dim() == 3:
        p, n = qkv.shape[0], qkv.shape[1]
        _check(qkv, "qkv", torch.float32, (p, n, width))
        return n, p, n * width
    n = qkv.shape[0]
    _check(qkv, "qkv", torch.float32, (n, width))
    return n, 1, 0


class KernelTimes:
    """Time on the GPU per kernel wrapper, from events recorded around every call: the
    "wall time per token, then a profiler" checklist of the reference (docs/PROFILING.md:7-11)
    without leaving the process.  Switched on by RBITNET_KERNEL_TIMES=1 (the decode step is then
    launched kernel by kernel instead of replayed as a graph, so that every launch can be timed);
    the table goes to standard error when the process ends, or to whoever calls `report()`."""

    def __init__(self, by_shape: bool = False) -> None:
        """by_shape (RBITNET_KERNEL_TIMES=shapes): a row per wrapper and shapes of its first two
        tensors, so that the products of a layer can be told apart."""
        self.by_shape = by_shape
        self.events: Dict[str, List[Tuple[torch.cuda.Event, torch.cuda.Event]]] = {}

    def wrap(self, name: str, fn):
        def timed(*args, **kwargs):
            key = name
            if self.by_shape:
                shapes = [tuple(a.shape) for a in args if hasattr(a, "shape")][:2]
                key = f"{name} " + " x ".join("[" + ",".join(str(d) for d in sh) + "]" for sh in shapes)
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            try:
                return fn(*args, **kwargs)
            finally:
                end.record()
                self.events.setdefault(key, []).append((start, end))
        return timed

    def totals(self) -> Dict[str, Tuple[int, float]]:
        """name -> (calls, milliseconds); waits for the GPU."""
        torch.cuda.synchronize()
        return {name: (len(pairs), sum(a.elapsed_time(b) for a, b in pairs)) for name, pairs in self.events.items()}

    def reset(self) -> None:
        self.events.clear()

    def report(self) -> str:
        totals = self.totals()
        whole = sum(ms for _, ms in totals.values()) or 1.0
        width = max([32] + [len(name) for name in totals])
        lines = [f"{'kernel':{width}} {'calls':>8} {'total ms':>10} {'mean us':>9} {'share':>6}"]
        for name, (calls, ms) in sorted(totals.items(), key=lambda kv: -kv[1][1]):
            lines.append(f"{name:{width}} {calls:8d} {ms:10.3f} {ms * 1e3 / max(1, calls):9.1f} {ms / whole:6.1%}")
        return "\n".join(lines)


TIMED_OPS = ("embed_gather", "add_rmsnorm", "rope_kv_write", "swiglu", "gemm_generic", "gemm_bf16", "gemm_bf16_terms",
             "gemm_bf16_few", "attention_generic", "attention_prefill_bf16", "attention_decode_bf16",
             "attention_decode_fused_bf16", "sample")


class Kernels:
    """The loaded library.  Methods check operand shapes on the host before a launch, so
    that a kernel never sees sizes other than the ones its grid assumes."""

    def __init__(self, path: Optional[str] = None):
        if not torch.cuda.is_available():
            raise KernelError("no GPU visible: rbitnet_amd runs on an MI355X (gfx950) only and has no CPU fallback")
        path = path or _build.ensure_built()
        try:
            self._lib = ctypes.CDLL(path)
        except OSError as e:
            raise KernelError(f"cannot load the HIP kernel library {path}: {e}") from None
        self.path = path
        L = self._lib
        L.rb_last_error.restype = ctypes.c_char_p
        sig = {
            "rb_embed_gather": [_P, _I, _P, _P, _I, _I, _P],
            "rb_add_rmsnorm": [_P, _P, _I, ctypes.c_longlong, _P, _F, _P, _I, _I, _P, _I, _P],
            "rb_rope_kv_write": [_P, _I, ctypes.c_longlong, _P, _P, _I, _P, _P, _P, _I, _P, _P, _P, _I, _I, _I, _I, _I, _P],
            "rb_swiglu": [_P, _P, _I, _I, _I, _P],
            "rb_gemm_generic": [_P, _P, _I, _P, _I, _I, _I, _I, _I, _P],
            "rb_gemm_bf16": [_P, _P, _I, _P, _I, _I, _I, _I, _I, _P, _P],
            "rb_gemm_bf16_few": [_P, _P, _F, _P, _P, _I, _P, _I, _I, _P, _P, _P, _I, _I, _I, _P],
            "rb_gemm_bf16_few_ok": [_I, _I, _I],
            "rb_gemm_bf16_terms_count": [_I, _I, _I],
            "rb_gemm_bf16_terms": [_P, _P, _I, _P, _I, _I, _I, _P],
            "rb_attention_generic": [_P, _P, _P, _P, _I, _P, _P, _P, _I, _I, _I, _I, _I, _F, _I, _P],
            "rb_attention_prefill_bf16": [_P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _F, _I, _P],
            "rb_attention_decode_bf16": [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _F, _I, _I, _P, _P],
            "rb_attention_decode_fused_bf16": [_P, _I, ctypes.c_longlong, _P, _P, _I, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _F, _I, _I,
                                               _P, _P],
            "rb_sample": [_P, _I, _I, _P, _P, _P, _P, _P],
            "rb_fill_normal": [_P, _I, ctypes.c_longlong, ctypes.c_ulonglong, ctypes.c_double, ctypes.c_double, _P],
            "rb_place_rows": [_P, _I, _P, _I, _I] + [ctypes.c_longlong] * 6 + [_P],
            "rb_probe_read": [_P, ctypes.c_longlong, _I, _I, _P, _P],
            "rb_probe_mfma": [_I, _I, _P, _P],
        }
        for name, args in sig.items():
            fn = getattr(L, name)
            fn.argtypes = args
            fn.restype = _I
        L.rb_plan_begin.argtypes, L.rb_plan_begin.restype = [], _P
        L.rb_plan_end.argtypes, L.rb_plan_end.restype = [_P], _I
        L.rb_plan_calls.argtypes, L.rb_plan_calls.restype = [_P], _I
        L.rb_plan_replay.argtypes, L.rb_plan_replay.restype = [_P, _P], _I
        L.rb_plan_free.argtypes, L.rb_plan_free.restype = [_P], None
        L.rb_gemm_workspace_floats.argtypes = [_I, _I, _I, _I]
        L.rb_gemm_workspace_floats.restype = ctypes.c_longlong
        L.rb_sample_workspace_bytes.argtypes = [_I, _I]
        L.rb_sample_workspace_bytes.restype = _I
        self.page_size = int(L.rb_page_size())
        self.times: Optional[KernelTimes] = None
        if os.environ.get("RBITNET_KERNEL_TIMES", "") in ("1", "true", "yes", "shapes"):
            self.times = KernelTimes(by_shape=os.environ["RBITNET_KERNEL_TIMES"] == "shapes")
            for name in TIMED_OPS:
                setattr(self, name, self.times.wrap(name, getattr(self, name)))
            atexit.register(lambda: print(self.times.report(), file=sys.stderr, flush=True))
        self.device_index = int(torch.cuda.current_device())
        self.n_compute_units = int(torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count)

    # ------------------------------------------------------------------ helpers
    def _stream(self) -> int:
        """torch's current HIP stream of this GPU, as a raw handle.  Asked for at every launch (a
        step that is being captured runs on another stream than the one before it), through torch's
        own fast path where it has one: `torch.cuda.current_stream()` builds a Python object at
        8 us a call, a third of what a launch costs on the host."""
        if _RAW_STREAM is not None:
            return _RAW_STREAM(self.device_index)
        return torch.cuda.current_stream().cuda_stream

    def _ok(self, rc: int) -> None:
        if rc != 0:
            raise KernelError(self._lib.rb_last_error().decode("utf-8", "replace"))

    # ------------------------------------------------------------------ ops
    def embed_gather(self, table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor) -> None:
        n, width = out.shape
        _check(table, "table")
        _check(ids, "ids", torch.int32, (n,))
        _check(out, "out", torch.float32)
        if table.shape[1] != width:
            raise KernelError("embedding width mismatch")
        self._ok(self._lib.rb_embed_gather(_ptr(table), dtype_code(table.dtype), _ptr(ids), _ptr(out), n, width,
                                           self._stream()))

    def add_rmsnorm(self, x: torch.Tensor, delta: Optional[torch.Tensor], gain: torch.Tensor, eps: float,
                    rows: Optional[torch.Tensor], out: torch.Tensor) -> None:
        n_rows, width = out.shape
        _check(x, "x", torch.float32)
        if x.shape[1] != width:
            raise KernelError("norm width mismatch")
        n_terms, term_stride = 1, 0
        if delta is not None:
            if delta.dim() == 3:            # several terms, to be added up first
                n_terms, term_stride = delta.shape[0], x.numel()
                _check(delta, "delta", torch.float32, (n_terms,) + tuple(x.shape))
            else:
                _check(delta, "delta", torch.float32, x.shape)
        _check(gain, "gain", torch.float32, (width,))
        if rows is not None:
            _check(rows, "rows", torch.int32, (n_rows,))
        elif x.shape[0] != n_rows:
            raise KernelError("norm row count mismatch")
        _check(out, "out")
        self._ok(self._lib.rb_add_rmsnorm(_ptr(x), _ptr(delta), n_terms, term_stride, _ptr(gain), float(eps),
                                          _ptr(rows), n_rows, width, _ptr(out), dtype_code(out.dtype),
                                          self._stream()))

    def rope_kv_write(self, qkv, cos, sin, style, q_out, k_pages, v_pages, tok_pos, tok_seq, block_table,
                      n_heads, n_kv, head_dim) -> None:
        n, n_terms, term_stride = _terms(qkv, (n_heads + 2 * n_kv) * head_dim)
        _check(q_out, "q_out", None, (n, n_heads, head_dim))
        _check(tok_pos, "tok_pos", torch.int32, (n,))
        _check(tok_seq, "tok_seq", torch.int32, (n,))
        _check(block_table, "block_table", torch.int32)
        if cos is not None:
            _check(cos, "cos", torch.float32)
            _check(sin, "sin", torch.float32, cos.shape)
            if cos.shape[1] != head_dim // 2:
                raise KernelError("angle table width mismatch")
        if k_pages is not None:
            _check(k_pages, "k_pages", q_out.dtype)
            _check(v_pages, "v_pages", q_out.dtype, k_pages.shape)
            if tuple(k_pages.shape[1:]) != (n_kv, self.page_size, head_dim):
                raise KernelError(f"cache pages have shape {tuple(k_pages.shape)}, expected "
                                  f"[*, {n_kv}, {self.page_size}, {head_dim}]")
        self._ok(self._lib.rb_rope_kv_write(_ptr(qkv), n_terms, term_stride, _ptr(cos), _ptr(sin), int(style),
                                            _ptr(q_out), _ptr(k_pages), _ptr(v_pages), dtype_code(q_out.dtype),
                                            _ptr(tok_pos), _ptr(tok_seq),
                                            _ptr(block_table), block_table.shape[1], n, n_heads, n_kv, head_dim,
                                            self._stream()))

    def swiglu(self, gu: torch.Tensor, out: torch.Tensor) -> None:
        n, ff = out.shape
        _check(gu, "gu", torch.float32, (n, 2 * ff))
        _check(out, "out")
        self._ok(self._lib.rb_swiglu(_ptr(gu), _ptr(out), dtype_code(out.dtype), n, ff, self._stream()))

    def gemm_generic(self, a: torch.Tensor, w: torch.Tensor, c: torch.Tensor, w_frag: bool = False) -> None:
        """w_frag: w [N, K] (float32) is stored fragment-major (`place_rows(..., frag=True)` writes that)."""
        m, k = a.shape
        n = w.shape[0]
        _check(a, "a")
        _check(w, "w", a.dtype, (n, k))
        _check(c, "c", None, (m, n))
        self._ok(self._lib.rb_gemm_generic(_ptr(a), _ptr(w), int(bool(w_frag)), _ptr(c), dtype_code(a.dtype),
                                           dtype_code(c.dtype), m, n, k, self._stream()))

    def gemm_bf16(self, a: torch.Tensor, w: torch.Tensor, c: torch.Tensor, epilogue: int = 0,
                  w_frag: bool = False) -> None:
        """w_frag: w [N, K] is stored fragment-major (`place_rows(..., frag=True)` writes that)."""
        m, k = a.shape
        n = w.shape[0]
        _check(a, "a", torch.bfloat16)
        _check(w, "w", torch.bfloat16, (n, k))
        _check(c, "c", None, (m, n // 2 if epilogue == 1 else n))
        need = int(self._lib.rb_gemm_workspace_floats(m, n, k, int(epilogue)))
        workspace = torch.empty(need, dtype=torch.float32, device=a.device) if need else None
        self._ok(self._lib.rb_gemm_bf16(_ptr(a), _ptr(w), int(bool(w_frag)), _ptr(c), dtype_code(c.dtype), int(epilogue),
                                        m, n, k, _ptr(workspace), self._stream()))

    def gemm_bf16_terms_count(self, m: int, n: int, k: int) -> int:
        return int(self._lib.rb_gemm_bf16_terms_count(int(m), int(n), int(k)))

    def gemm_bf16_terms(self, a: torch.Tensor, w: torch.Tensor, w_frag: bool = False) -> torch.Tensor:
        """a w^T as float32 terms [P, M, N] to be added up in their order: what the K slices of
        the kernel for these sizes computed (P = 1: the product itself)."""
        m, k = a.shape
        n = w.shape[0]
        _check(a, "a", torch.bfloat16)
        _check(w, "w", torch.bfloat16, (n, k))
        terms = torch.empty((int(self._lib.rb_gemm_bf16_terms_count(m, n, k)), m, n), dtype=torch.float32,
                            device=a.device)
        self._ok(self._lib.rb_gemm_bf16_terms(_ptr(a), _ptr(w), int(bool(w_frag)), _ptr(terms), m, n, k, self._stream()))
        return terms

    def gemm_bf16_few_ok(self, m: int, n: int, k: int) -> bool:
        """Whether gemm_bf16_few takes these sizes (1..16 tokens)."""
        return bool(self._lib.rb_gemm_bf16_few_ok(int(m), int(n), int(k)))

    def gemm_bf16_few(self, a: torch.Tensor, w: torch.Tensor, c: torch.Tensor, epilogue: int = 0,
                      squares: Optional[torch.Tensor] = None, eps: float = 0.0, rows: Optional[torch.Tensor] = None,
                      gain: Optional[torch.Tensor] = None, gained: Optional[torch.Tensor] = None,
                      squares_out: Optional[torch.Tensor] = None, w_frag: bool = False) -> None:
        """The product of 1..16 tokens with its neighbours folded in.
        squares [*, ceil(K / 16)]: a holds rows times a norm's gain and squares the sums of squares
        of the rows themselves; the product is scaled to that of the RMS-normalised rows (eps).
        rows: the tokens are these rows of a (and of squares).
        epilogue 2: c (float32) += product.  epilogue 3: the same, and gained [M, N] =
        bf16(c * gain), squares_out [M, ceil(N / 16)] = sums of c^2, for the norm that follows."""
        n, k = w.shape
        _check(a, "a", torch.bfloat16)
        if a.dim() != 2 or a.shape[1] != k:
            raise KernelError(f"a must have rows of {k} values, found {tuple(a.shape)}")
        m = a.shape[0] if rows is None else rows.shape[0]
        if rows is not None:
            _check(rows, "rows", torch.int32, (m,))
        if squares is not None:
            _check(squares, "squares", torch.float32, (a.shape[0], (k + 15) // 16))
        _check(w, "w", torch.bfloat16, (n, k))
        _check(c, "c", torch.float32 if epilogue >= 2 else None, (m, n // 2 if epilogue == 1 else n))
        if epilogue == 3:
            _check(gain, "gain", torch.float32, (n,))
            _check(gained, "gained", torch.bfloat16, (m, n))
            _check(squares_out, "squares_out", torch.float32, (m, (n + 15) // 16))
        self._ok(self._lib.rb_gemm_bf16_few(_ptr(a), _ptr(squares), float(eps), _ptr(rows), _ptr(w), int(bool(w_frag)),
                                            _ptr(c), dtype_code(c.dtype), int(epilogue), _ptr(gain), _ptr(gained),
                                            _ptr(squares_out), m, n, k, self._stream()))

    def attention_generic(self, q, k_pages, v_pages, out, tok_pos, tok_seq, block_table, n_heads, n_kv, head_dim,
                          scale, window) -> None:
        n = q.shape[0]
        _check(q, "q", None, (n, n_heads, head_dim))
        _check(k_pages, "k_pages", q.dtype)
        _check(v_pages, "v_pages", q.dtype, k_pages.shape)
        if tuple(k_pages.shape[1:]) != (n_kv, self.page_size, head_dim):
            raise KernelError("cache pages do not match the head counts")
        _check(out, "out", q.dtype, (n, n_heads * head_dim))
        _check(tok_pos, "tok_pos", torch.int32, (n,))
        _check(tok_seq, "tok_seq", torch.int32, (n,))
        _check(block_table, "block_table", torch.int32)
        self._ok(self._lib.rb_attention_generic(_ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(out), dtype_code(q.dtype),
                                                _ptr(tok_pos), _ptr(tok_seq), _ptr(block_table),
                                                block_table.shape[1], n, n_heads, n_kv, head_dim, float(scale),
                                                int(window or 0), self._stream()))

    def attention_prefill_bf16(self, q, k_pages, v_pages, out, cu_seqlens, past_len, block_table, n_seqs,
                               max_q_len, n_heads, n_kv, head_dim, scale, window) -> None:
        n = q.shape[0]
        _check(q, "q", torch.bfloat16, (n, n_heads, head_dim))
        _check(k_pages, "k_pages", torch.bfloat16)
        _check(v_pages, "v_pages", torch.bfloat16, k_pages.shape)
        if tuple(k_pages.shape[1:]) != (n_kv, self.page_size, head_dim):
            raise KernelError("cache pages do not match the head counts")
        _check(out, "out", torch.bfloat16, (n, n_heads * head_dim))
        _check(cu_seqlens, "cu_seqlens", torch.int32, (n_seqs + 1,))
        _check(past_len, "past_len", torch.int32, (n_seqs,))
        _check(block_table, "block_table", torch.int32)
        self._ok(self._lib.rb_attention_prefill_bf16(_ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(out),
                                                     _ptr(cu_seqlens), _ptr(past_len), _ptr(block_table),
                                                     block_table.shape[1], n_seqs, int(max_q_len), n_heads, n_kv,
                                                     head_dim, float(scale), int(window or 0), self._stream()))

    def attention_decode_bf16(self, q, k_pages, v_pages, out, tok_pos, block_table, n_heads, n_kv, head_dim,
                              scale, window, n_splits, workspace) -> None:
        n = q.shape[0]
        _check(q, "q", torch.bfloat16, (n, n_heads, head_dim))
        _check(k_pages, "k_pages", torch.bfloat16)
        _check(v_pages, "v_pages", torch.bfloat16, k_pages.shape)
        if tuple(k_pages.shape[1:]) != (n_kv, self.page_size, head_dim):
            raise KernelError("cache pages do not match the head counts")
        _check(out, "out", torch.bfloat16, (n, n_heads * head_dim))
        _check(tok_pos, "tok_pos", torch.int32, (n,))
        _check(block_table, "block_table", torch.int32)
        _check(workspace, "workspace", torch.float32)
        if workspace.numel() < n * n_heads * n_splits * (head_dim + 2):
            raise KernelError("decode attention workspace too small")
        self._ok(self._lib.rb_attention_decode_bf16(_ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(out), _ptr(tok_pos),
                                                    _ptr(block_table), block_table.shape[1], n, n_heads, n_kv,
                                                    head_dim, float(scale), int(window or 0), int(n_splits),
                                                    _ptr(workspace), self._stream()))

    def attention_decode_fused_bf16(self, qkv, cos, sin, style, k_pages, v_pages, out, tok_pos, block_table,
                                    n_heads, n_kv, head_dim, scale, window, n_splits, workspace) -> None:
        n, n_terms, term_stride = _terms(qkv, (n_heads + 2 * n_kv) * head_dim)
        if cos is not None:
            _check(cos, "cos", torch.float32)
            _check(sin, "sin", torch.float32, cos.shape)
            if cos.shape[1] != head_dim // 2:
                raise KernelError("angle table width mismatch")
        _check(k_pages, "k_pages", torch.bfloat16)
        _check(v_pages, "v_pages", torch.bfloat16, k_pages.shape)
        if tuple(k_pages.shape[1:]) != (n_kv, self.page_size, head_dim):
            raise KernelError("cache pages do not match the head counts")
        _check(out, "out", torch.bfloat16, (n, n_heads * head_dim))
        _check(tok_pos, "tok_pos", torch.int32, (n,))
        _check(block_table, "block_table", torch.int32)
        _check(workspace, "workspace", torch.float32)
        if workspace.numel() < n * n_heads * n_splits * (head_dim + 2):
            raise KernelError("decode attention workspace too small")
        self._ok(self._lib.rb_attention_decode_fused_bf16(
            _ptr(qkv), n_terms, term_stride, _ptr(cos), _ptr(sin), int(style), _ptr(k_pages), _ptr(v_pages), _ptr(out),
            _ptr(tok_pos),
            _ptr(block_table), block_table.shape[1], n, n_heads, n_kv, head_dim, float(scale), int(window or 0),
            int(n_splits), _ptr(workspace), self._stream()))

    def sample(self, logits: torch.Tensor, temperature: Optional[torch.Tensor], u: Optional[torch.Tensor],
               tokens: torch.Tensor, workspace: Optional[torch.Tensor] = None) -> None:
        n, vocab = logits.shape
        _check(logits, "logits", torch.float32)
        if temperature is not None:
            _check(temperature, "temperature", torch.float32, (n,))
            _check(u, "u", torch.float32, (n,))
        _check(tokens, "tokens", torch.int32, (n,))
        need = int(self._lib.rb_sample_workspace_bytes(n, vocab))
        if workspace is None:
            workspace = torch.empty((need + 7) // 8, dtype=torch.int64, device=logits.device)
        _check(workspace, "workspace", torch.int64)
        if workspace.numel() * 8 < need:
            raise KernelError("sampling workspace too small")
        self._ok(self._lib.rb_sample(_ptr(logits), n, vocab, _ptr(temperature), _ptr(u), _ptr(tokens),
                                     _ptr(workspace), self._stream()))

    # ------------------------------------------------------------------ recorded steps
    def plan_begin(self) -> int:
        """From here to `plan_end` every launch of this thread is noted as well as issued; returns
        the plan's handle."""
        plan = self._lib.rb_plan_begin()
        if not plan:
            raise KernelError(self._lib.rb_last_error().decode("utf-8", "replace"))
        return plan

    def plan_end(self, plan: int) -> int:
        """Ends the recording; returns the number of launches the plan holds."""
        self._ok(self._lib.rb_plan_end(plan))
        return int(self._lib.rb_plan_calls(plan))

    def plan_replay(self, plan: int) -> None:
        """Issues the plan's launches again on torch's current stream, with the arguments they were
        recorded with: the memory those name must still be the step's own."""
        self._ok(self._lib.rb_plan_replay(plan, self._stream()))

    def plan_free(self, plan: int) -> None:
        self._lib.rb_plan_free(plan)

    # ------------------------------------------------------------------ load time
    def fill_normal(self, out: torch.Tensor, key: int, mean: float, std: float) -> None:
        """out[i] = mean + std * (the standard normal number that (key, i) fixes)."""
        _check(out, "out")
        self._ok(self._lib.rb_fill_normal(_ptr(out), dtype_code(out.dtype), out.numel(), int(key) & (2**64 - 1),
                                          float(mean), float(std), self._stream()))

    def place_rows(self, src: torch.Tensor, dst: torch.Tensor, row0: int = 0, block: Optional[int] = None,
                   period: Optional[int] = None, frag: bool = False) -> None:
        """Row r of src goes, cast to dst's dtype, to row row0 + (r // block) * period + r % block
        of dst (block: all rows, so that they follow one another from row0).  frag: dst is stored
        fragment-major (the matrix-core products' other layout of W; rows % 16 == 0, width % 32 == 0)."""
        _check(src, "src")
        _check(dst, "dst")
        if src.dim() != 2 or dst.dim() != 2 or src.shape[1] != dst.shape[1]:
            raise KernelError(f"place_rows: {tuple(src.shape)} does not fit into {tuple(dst.shape)}")
        n = src.shape[0]
        block = max(1, n) if block is None else int(block)
        period = block if period is None else int(period)
        self._ok(self._lib.rb_place_rows(_ptr(src), dtype_code(src.dtype), _ptr(dst), dtype_code(dst.dtype),
                                         int(bool(frag)), n, src.shape[1], dst.shape[0], int(row0), block, period,
                                         self._stream()))

    # ------------------------------------------------------------------ probes
    def probe_read(self, buf: torch.Tensor, sink: torch.Tensor, blocks: int = 2048, pieces: bool = False) -> None:
        """Reads every byte of `buf` once with `blocks` workgroups (see probe.hip).  pieces: every
        workgroup walks pieces of its own with non-temporal loads, as the decode products do."""
        _check(buf, "buf")
        _check(sink, "sink", torch.float32)
        nbytes = buf.numel() * buf.element_size()
        if nbytes % 16 != 0 or buf.data_ptr() % 16 != 0:
            raise KernelError("probe buffer must be 16-byte aligned and a multiple of 16 bytes long")
        self._ok(self._lib.rb_probe_read(_ptr(buf), nbytes, int(blocks), int(bool(pieces)), _ptr(sink), self._stream()))

    def probe_mfma(self, waves: int, iters: int, sink: torch.Tensor) -> float:
        """Runs the MFMA loop; returns the floating-point operations it performs."""
        _check(sink, "sink", torch.float32)
        self._ok(self._lib.rb_probe_mfma(int(waves), int(iters), _ptr(sink), self._stream()))
        return float(waves) * iters * 4 * 2 * 32 * 32 * 16


_lock = threading.Lock()
_instance: Optional[Kernels] = None


def kernels() -> Kernels:
    """The process-wide library, loaded (and built, if it is not) at first use."""
    global _instance
    with _lock:
        if _instance is None:
            _instance = Kernels()
        return _instance
