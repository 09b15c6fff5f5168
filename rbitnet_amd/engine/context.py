"""What a step's kernels need to know about its batch: ONE layout, declared once, built on
the host and sent to the GPU in one copy.

Tokens of all sequences are packed one after another ([T] rows, no padding):
sequence b holds rows cu_seqlens[b] .. cu_seqlens[b+1], at positions
past_len[b], past_len[b] + 1, ...

A `StepContext` is made for given sizes (sequences, tokens, asked rows, widths of the page
tables) and owns a pinned host buffer and a device buffer of that layout; `fill(batch)`
writes the host side and copies it over.  A step that is launched kernel by kernel makes
a context for its batch and fills it once; a captured decode step keeps one context and
fills it again before every replay, so that the kernels in the graph always read the
same addresses.  Both are this class: an array that a part needs per step is declared in
one place, `declare_step_array`, and is there in both.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

# tests may force a number of splits of decode attention (None: the built-in choice)
FORCED_DECODE_SPLITS: Optional[int] = None


def split_bucket(max_kv_len: int) -> int:
    """1, 2, 4, 8 or 16 by the longest context of the batch: about eight pages of 64 keys per
    split (a workgroup walks four pages at a time; a page costs far less than the second
    launch that combines splits, so short contexts are not split at all)."""
    pages = (max(1, int(max_kv_len)) + 63) // 64
    bucket = 1
    while bucket < 16 and bucket * 2 <= pages // 8:
        bucket *= 2
    return bucket


def bucket_max_pages(bucket: int) -> int:
    """The most pages a sequence can hold while its batch is in this bucket (None: no bound)."""
    return None if bucket >= 16 else 16 * bucket - 1


def decode_splits(n_seqs: int, n_kv_heads: int, bucket: int, n_compute_units: int) -> int:
    """Into how many workgroups the pages of one (sequence, kv head) are dealt in decode
    attention: what the context length asks for (`split_bucket`), but no more than gives
    every compute unit about one workgroup (every split adds to the combination)."""
    if FORCED_DECODE_SPLITS:
        return max(1, int(FORCED_DECODE_SPLITS))
    return max(1, min(int(bucket), 16, n_compute_units // max(1, n_seqs * max(1, n_kv_heads))))


@dataclass
class StepBatch:
    """One step as the host knows it."""
    slots: Sequence[int]
    past_lens: Sequence[int]
    tokens: Sequence[Sequence[int]]            # per sequence, the tokens to run
    rows: Sequence[int]                        # packed rows whose logits are asked for
    block_tables: Dict[int, List[List[int]]]   # storage group -> per sequence, its pages
    temperatures: Optional[Sequence[float]] = None
    uniforms: Optional[Sequence[float]] = None


@dataclass
class _StepArray:
    name: str
    dtype: str                                           # "int32" or "float32"
    size: Callable[[int, int], int]                      # (sequences, tokens) -> elements
    fill: Callable[[StepBatch], np.ndarray]


_EXTRA_ARRAYS: Dict[str, _StepArray] = {}


def declare_step_array(name: str, dtype: str, size: Callable[[int, int], int],
                       fill: Callable[[StepBatch], np.ndarray]) -> None:
    """A per-step array of a part's own: `fill(batch)` computes it on the host for every
    step, kernels find it at `ctx.extra[name]` (a device tensor of `size(sequences, tokens)`
    elements), in steps launched one by one and in captured ones alike."""
    if dtype not in ("int32", "float32"):
        raise ValueError("a step array holds int32 or float32")
    _EXTRA_ARRAYS[name] = _StepArray(name, dtype, size, fill)


def forget_step_array(name: str) -> None:
    _EXTRA_ARRAYS.pop(name, None)


class StepContext:
    def __init__(self, device, n_seqs: int, n_tokens: int, n_rows: int, table_widths: Dict[int, int],
                 bucket: Optional[int] = None, *, n_compute_units: int):
        """bucket: the split bucket of decode attention when it must not follow the batch (a
        captured step's grid cannot change); None: from each batch's longest context."""
        b, t = int(n_seqs), int(n_tokens)
        self.device = device
        self.n_seqs, self.n_tokens, self.n_rows = b, t, int(n_rows)
        self.fixed_bucket = bucket
        self.bucket = bucket or 1
        self.n_compute_units = int(n_compute_units)
        # ---- the layout: every array of a step, once
        fields: List[Tuple[str, str, int, Optional[Tuple[int, ...]]]] = [
            ("token_ids", "int32", t, None), ("tok_pos", "int32", t, None), ("tok_seq", "int32", t, None),
            ("cu_seqlens", "int32", b + 1, None), ("past_len", "int32", b, None), ("slots", "int32", b, None),
            ("rows", "int32", self.n_rows, None),
            ("temperature", "float32", b, None), ("uniform", "float32", b, None),
        ]
        for key, width in table_widths.items():
            fields.append((("table", key), "int32", b * width, (b, width)))
        for arr in _EXTRA_ARRAYS.values():
            fields.append((("extra", arr.name), arr.dtype, int(arr.size(b, t)), None))
        total = sum(n for _, _, n, _ in fields)
        self._host = torch.zeros(max(1, total), dtype=torch.int32)
        if torch.device(device).type == "cuda":
            self._host = self._host.pin_memory()
        self._dev = torch.empty(max(1, total), dtype=torch.int32, device=device)
        h_all = self._host.numpy()
        self._h: Dict = {}
        self.block_tables: Dict[int, torch.Tensor] = {}
        self.extra: Dict[str, torch.Tensor] = {}
        off = 0
        for name, dtype, n, shape in fields:
            d, h = self._dev[off:off + n], h_all[off:off + n]
            off += n
            if dtype == "float32":
                d, h = d.view(torch.float32), h.view(np.float32)
            if shape is not None:
                d, h = d.view(shape), h.reshape(shape)
            self._h[name] = h
            if isinstance(name, tuple) and name[0] == "table":
                self.block_tables[name[1]] = d
            elif isinstance(name, tuple):
                self.extra[name[1]] = d
            else:
                setattr(self, name, d)
        # ---- what the host keeps of the current batch
        self.q_lens: List[int] = []
        self.max_q_len = 0
        self.max_kv_len = 0
        self.host_slots: List[int] = []
        self.host_past: List[int] = []
        self._workspaces: Dict[Tuple[int, int, int, int], Tuple] = {}
        self._copied: Optional[torch.cuda.Event] = None      # the last copy of the host buffer to the device

    @classmethod
    def for_batch(cls, device, batch: StepBatch, n_compute_units: int) -> "StepContext":
        widths = {key: max(1, max(len(r) for r in table)) for key, table in batch.block_tables.items()}
        ctx = cls(device, len(batch.slots), sum(len(t) for t in batch.tokens), len(batch.rows), widths,
                  n_compute_units=n_compute_units)
        ctx.fill(batch)
        return ctx

    def fill(self, batch: StepBatch) -> None:
        """Writes the batch into the layout and copies it to the GPU (one copy)."""
        if self._copied is not None:
            self._copied.synchronize()        # the copy before this one has read the host buffer
        q_lens = [len(t) for t in batch.tokens]
        b, t = len(batch.slots), int(sum(q_lens))
        if b != self.n_seqs or t != self.n_tokens or len(batch.rows) != self.n_rows:
            raise ValueError("the batch does not have the sizes this step layout was made for")
        h = self._h
        past = np.asarray(batch.past_lens, dtype=np.int32)
        h["token_ids"][:] = np.concatenate([np.asarray(x, dtype=np.int64) for x in batch.tokens]).astype(np.int32)
        tok_seq = np.repeat(np.arange(b, dtype=np.int32), q_lens)
        h["tok_seq"][:] = tok_seq
        cu = h["cu_seqlens"]
        cu[0] = 0
        np.cumsum(q_lens, out=cu[1:])
        h["tok_pos"][:] = np.arange(t, dtype=np.int32) - cu[tok_seq] + past[tok_seq]
        h["past_len"][:] = past
        h["slots"][:] = np.asarray(batch.slots, dtype=np.int32)
        h["rows"][:] = np.asarray(batch.rows, dtype=np.int32)
        h["temperature"][:] = 0.0 if batch.temperatures is None else np.asarray(batch.temperatures, dtype=np.float32)
        h["uniform"][:] = 0.0 if batch.uniforms is None else np.asarray(batch.uniforms, dtype=np.float32)
        for key, table in batch.block_tables.items():
            dst = h[("table", key)]
            for i, pages in enumerate(table):
                n = len(pages)
                if n > dst.shape[1]:
                    raise ValueError("a sequence holds more pages than the step layout has room for")
                dst[i, :n] = pages
        for arr in _EXTRA_ARRAYS.values():
            h[("extra", arr.name)][:] = arr.fill(batch)
        self.q_lens = q_lens
        self.max_q_len = max(q_lens)
        self.max_kv_len = max(p + q for p, q in zip(batch.past_lens, q_lens))
        self.host_slots = list(batch.slots)
        self.host_past = list(batch.past_lens)
        if self.fixed_bucket is None:
            self.bucket = split_bucket(self.max_kv_len)
        self._dev.copy_(self._host, non_blocking=True)
        if self._host.is_pinned():
            if self._copied is None:
                self._copied = torch.cuda.Event()
            self._copied.record()

    def decode_workspace(self, n_heads: int, head_dim: int, n_kv_heads: int = 1) -> Tuple:
        """Split count and scratch for decode attention: enough workgroups to fill the
        GPU, whatever the context length (each split strides over the pages)."""
        n_splits = decode_splits(self.n_seqs, n_kv_heads, self.bucket, self.n_compute_units)
        key = (n_heads, head_dim, n_kv_heads, n_splits)
        if key not in self._workspaces:
            ws = torch.empty(self.n_seqs * n_heads * n_splits * (head_dim + 2), dtype=torch.float32,
                             device=self.device)
            self._workspaces[key] = (n_splits, ws)
        return self._workspaces[key]
