"""The decode step as a HIP graph: one token per sequence in, the next token per
sequence out, replayed with nothing but one small host-to-device copy in between.

A decode step of a 32-layer model is some three hundred kernel launches; issued one by
one from Python they cost more host time than the GPU needs to run them.  The launches of
one step depend only on the number of sequences, so they are captured once per batch size
into a graph whose kernels read everything that changes (tokens, positions, page tables,
temperatures, uniform numbers) from fixed device buffers.

No memset is recorded into the graph (the buffers are written by a copy issued before
each replay, outside the graph), and only this library's kernels run inside it.
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from ..cache.pages import pages_for
from .context import decode_splits


class _StaticContext:
    """Has the attributes of `StepContext`, but every device tensor is a fixed view into
    one buffer that `DecodeGraph.run` refreshes before each replay."""

    def __init__(self, device, n_seqs: int, group_keys: Sequence[int], table_width: int, bucket: int = 16):
        b = n_seqs
        self.device = device
        self.bucket = bucket             # of the longest context this graph is replayed for (context.split_bucket)
        self.n_seqs = b
        self.n_tokens = b
        self.max_q_len = 1
        self.q_lens = [1] * b
        self.table_width = table_width
        n_int = 4 * b + (b + 1) + b + b + len(group_keys) * b * table_width
        self.n_float = 2 * b
        self.host = torch.zeros(n_int + self.n_float, dtype=torch.int32).pin_memory()
        self.dev = torch.zeros(n_int + self.n_float, dtype=torch.int32, device=device)
        self.h = self.host.numpy()
        off = 0

        def take(n: int) -> Tuple[torch.Tensor, np.ndarray]:
            nonlocal off
            out = (self.dev[off:off + n], self.h[off:off + n])
            off += n
            return out

        self.token_ids, self.h_tokens = take(b)
        self.tok_pos, self.h_pos = take(b)
        self.past_len, self.h_past = take(b)
        self.slots, self.h_slots = take(b)
        self.tok_seq, h_seq = take(b)
        self.cu_seqlens, h_cu = take(b + 1)
        self.rows, h_rows = take(b)
        h_seq[:] = np.arange(b)
        h_cu[:] = np.arange(b + 1)
        h_rows[:] = np.arange(b)
        self.block_tables: Dict[int, torch.Tensor] = {}
        self.h_tables: Dict[int, np.ndarray] = {}
        for key in group_keys:
            d, h = take(b * table_width)
            self.block_tables[key] = d.view(b, table_width)
            self.h_tables[key] = h.reshape(b, table_width)
        fd, fh = take(2 * b)
        fdev = fd.view(torch.float32)
        self.temperature, self.uniform = fdev[:b], fdev[b:]
        fhost = fh.view(np.float32)
        self.h_temperature, self.h_uniform = fhost[:b], fhost[b:]
        self.host_slots: List[int] = [0] * b
        self.host_past: List[int] = [0] * b
        self.max_kv_len = 0
        self._workspaces: Dict[Tuple[int, int, int], Tuple] = {}

    def decode_workspace(self, n_heads: int, head_dim: int, n_kv_heads: int = 1):
        key = (n_heads, head_dim, n_kv_heads)
        if key not in self._workspaces:
            n_splits = decode_splits(self.n_seqs, n_kv_heads, self.bucket)
            ws = torch.empty(self.n_seqs * n_heads * n_splits * (head_dim + 2), dtype=torch.float32,
                             device=self.device)
            self._workspaces[key] = (n_splits, ws)
        return self._workspaces[key]

    def upload(self) -> None:
        self.dev.copy_(self.host, non_blocking=True)


class DecodeGraph:
    """One captured decode step for a fixed number of sequences and a fixed split count of
    decode attention (the grid of a captured launch cannot change)."""

    def __init__(self, engine, n_seqs: int, bucket: int = 16):
        self.engine = engine
        self.n_seqs = n_seqs
        width = max(1, pages_for(engine.max_seq_len))
        self.ctx = _StaticContext(engine.device, n_seqs, [id(g) for g in engine.cache.kv_groups], width, bucket)
        self.tokens_out = torch.zeros(n_seqs, dtype=torch.int32, device=engine.device)
        self.logits: Optional[torch.Tensor] = None
        self.graph: Optional[torch.cuda.CUDAGraph] = None

    def _fill(self, slots, tokens, temperatures, uniforms) -> None:
        c, cache = self.ctx, self.engine.cache
        past = [cache.length(s) for s in slots]
        c.h_tokens[:] = tokens
        c.h_pos[:] = past
        c.h_past[:] = past
        c.h_slots[:] = slots
        c.host_slots[:] = slots
        c.host_past[:] = past
        c.max_kv_len = max(past) + 1
        for g in cache.kv_groups:
            table = c.h_tables[id(g)]
            for i, s in enumerate(slots):
                pages = g.table.pages(s)
                n = len(pages)
                table[i, :n] = [p if p >= 0 else 0 for p in pages]
        c.h_temperature[:] = 0.0 if temperatures is None else temperatures
        c.h_uniform[:] = 0.0 if uniforms is None else uniforms
        c.upload()

    def _launch(self) -> None:
        eng, c = self.engine, self.ctx
        self.logits = eng.model.forward(c, eng.cache, c.rows)
        eng.lib.sample(self.logits, c.temperature, c.uniform, self.tokens_out)

    def run(self, slots, tokens, temperatures=None, uniforms=None) -> list:
        eng = self.engine
        q = [1] * self.n_seqs
        eng.cache.reserve(slots, q)
        self._fill(slots, tokens, temperatures, uniforms)
        if self.graph is None:
            # warm up on a side stream (allocations settle), then capture
            side = torch.cuda.Stream(device=eng.device)
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                self._launch()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                self._launch()
            self.graph = graph
        self.graph.replay()
        out = self.tokens_out.tolist()
        eng.cache.commit(slots, q)
        return out
