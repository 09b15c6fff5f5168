"""What a step's kernels need to know about its batch, built once per step on the host
and sent to the GPU in one copy.

Tokens of all sequences are packed one after another ([T] rows, no padding):
sequence b holds rows cu_seqlens[b] .. cu_seqlens[b+1], at positions
past_len[b], past_len[b] + 1, ...
"""
from __future__ import annotations

from typing import Dict, List, Sequence, Tuple

import numpy as np
import torch


def split_bucket(max_kv_len: int) -> int:
    """1, 2, 4, 8 or 16 by the longest context of the batch: about eight pages of 64 keys per
    split (a workgroup walks four pages at a time; a page costs far less than the second
    launch that combines splits, so short contexts are not split at all)."""
    pages = (max(1, int(max_kv_len)) + 63) // 64
    bucket = 1
    while bucket < 16 and bucket * 2 <= pages // 8:
        bucket *= 2
    return bucket


def decode_splits(n_seqs: int, n_kv_heads: int, bucket: int = 16) -> int:
    """Into how many workgroups the pages of one (sequence, kv head) are dealt in decode
    attention: what the context length asks for (`split_bucket`), but no more than gives
    every compute unit about one workgroup (every split adds to the combination)."""
    import os
    forced = os.environ.get("RBITNET_DECODE_SPLITS")
    if forced:
        return max(1, int(forced))
    return max(1, min(int(bucket), 16, 256 // max(1, n_seqs * max(1, n_kv_heads))))


class StepContext:
    def __init__(self, device, slots: Sequence[int], past_lens: Sequence[int], tokens: Sequence[Sequence[int]],
                 rows: Sequence[int], block_tables: Dict[int, List[List[int]]], n_kv_heads_hint: int = 1):
        self.device = device
        self.n_seqs = len(slots)
        q_lens = [len(t) for t in tokens]
        self.q_lens = q_lens
        self.n_tokens = int(sum(q_lens))
        self.max_q_len = max(q_lens)
        self.max_kv_len = max(p + q for p, q in zip(past_lens, q_lens))
        self.host_slots = list(slots)
        self.host_past = list(past_lens)
        b, t = self.n_seqs, self.n_tokens

        ids = np.concatenate([np.asarray(x, dtype=np.int64) for x in tokens]).astype(np.int32)
        tok_seq = np.repeat(np.arange(b, dtype=np.int32), q_lens)
        cu = np.zeros(b + 1, dtype=np.int32)
        np.cumsum(q_lens, out=cu[1:])
        tok_pos = (np.arange(t, dtype=np.int32) - cu[tok_seq] + np.asarray(past_lens, dtype=np.int32)[tok_seq])
        pieces = [ids, tok_pos.astype(np.int32), tok_seq, cu, np.asarray(past_lens, dtype=np.int32),
                  np.asarray(slots, dtype=np.int32), np.asarray(rows, dtype=np.int32)]
        tables = []
        for key, table in block_tables.items():
            arr = np.asarray(table, dtype=np.int32).reshape(b, -1)
            tables.append((key, arr.shape[1]))
            pieces.append(arr.reshape(-1))
        flat = np.concatenate(pieces)
        host = torch.from_numpy(flat)
        if torch.device(device).type == "cuda":
            host = host.pin_memory()
        dev = host.to(device, non_blocking=True)
        self._host_keepalive = host
        off = 0

        def take(n: int) -> torch.Tensor:
            nonlocal off
            out = dev[off:off + n]
            off += n
            return out

        self.token_ids = take(t)
        self.tok_pos = take(t)
        self.tok_seq = take(t)
        self.cu_seqlens = take(b + 1)
        self.past_len = take(b)
        self.slots = take(b)
        self.rows = take(len(rows))
        self.block_tables: Dict[int, torch.Tensor] = {}
        for key, width in tables:
            self.block_tables[key] = take(b * width).view(b, width)
        self._workspaces: Dict[Tuple[int, int, int], Tuple] = {}

    def decode_workspace(self, n_heads: int, head_dim: int, n_kv_heads: int = 1) -> Tuple:
        """Split count and scratch for decode attention: enough workgroups to fill the
        GPU, whatever the context length (each split strides over the pages)."""
        key = (n_heads, head_dim, n_kv_heads)
        if key not in self._workspaces:
            n_splits = decode_splits(self.n_seqs, n_kv_heads, split_bucket(self.max_kv_len))
            ws = torch.empty(self.n_seqs * n_heads * n_splits * (head_dim + 2), dtype=torch.float32,
                             device=self.device)
            self._workspaces[key] = (n_splits, ws)
        return self._workspaces[key]
