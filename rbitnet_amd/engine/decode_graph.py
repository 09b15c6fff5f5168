"""The decode step as a HIP graph: one token per sequence in, the next token per
sequence out, replayed with nothing but one small host-to-device copy in between.

A decode step of a 32-layer model is some three hundred kernel launches; issued one by
one from Python they cost more host time than the GPU needs to run them.  The launches of
one step depend only on the number of sequences, so they are captured once per batch size
into a graph whose kernels read everything that changes (tokens, positions, page tables,
temperatures, uniform numbers) from fixed device buffers.

No memset is recorded into the graph (the buffers are written by a copy issued before
each replay, outside the graph), and only this library's kernels run inside it.

A batch whose sequences end one by one would need a capture for every size on the way down.
Graphs are therefore captured for a ladder of sizes only (`graph_size`), and a batch runs in the
graph of the next size up: the rows beyond its own are idle rows, each a sequence of length 0 in
the cache's spare slot, whose token (id 0 at position 0) writes its key, value and state to the
spare page and the spare state and reads nothing else.  A live row's result does not depend on the
idle rows: every kernel of a step computes a row from that row's inputs alone.
"""
from __future__ import annotations

import weakref
from typing import Optional

import torch

from .context import StepBatch, StepContext, bucket_max_pages

GRAPH_SIZES = (1, 2, 3, 4, 6, 8, 12, 16, 24, 32, 48, 64)


def graph_size(n_seqs: int) -> int:
    """The size of the captured step that a batch of n sequences runs in: the next of 1, 2, 3, 4, 6,
    8, 12, 16, 24, 32, 48, 64, and multiples of 32 beyond, so that at most a third of the rows idle."""
    for size in GRAPH_SIZES:
        if n_seqs <= size:
            return size
    return (int(n_seqs) + 31) // 32 * 32


class DecodeGraph:
    """One captured decode step for a fixed number of sequences and a fixed split count of
    decode attention (the grid of a captured launch cannot change).  Its `StepContext` is made
    once, with page tables wide enough for the longest sequence the engine allows, and filled
    again before every replay."""

    def __init__(self, engine, n_seqs: int, bucket: int = 16):
        self.engine = weakref.proxy(engine)      # no cycle of references: the graphs go when the engine goes
        self.n_seqs = n_seqs
        # page tables as wide as a sequence of this graph can need: no longer than the engine
        # allows, than the cache has pages, or than the contexts of this split bucket reach
        width = min(engine.cache.pages_per_sequence(engine.max_seq_len), engine.cache.n_pages)
        if bucket_max_pages(bucket) is not None:
            width = min(width, bucket_max_pages(bucket))
        width = max(1, width)
        self.ctx = StepContext(engine.device, n_seqs, n_seqs, n_seqs,
                               {key: width for key in engine.cache.group_keys()}, bucket=bucket,
                               n_compute_units=engine.lib.n_compute_units)
        self.tokens_out = torch.zeros(n_seqs, dtype=torch.int32, device=engine.device)
        self.logits: Optional[torch.Tensor] = None           # of the captured launches: valid after a replay
        self.first_logits: Optional[torch.Tensor] = None     # of the step that ran before the capture
        self.graph: Optional[torch.cuda.CUDAGraph] = None

    def _fill(self, slots, tokens, temperatures, uniforms) -> None:
        cache = self.engine.cache
        idle = self.n_seqs - len(slots)
        past = [cache.length(s) for s in slots] + [0] * idle
        slots = list(slots) + [cache.spare_slot] * idle
        pad = lambda values: None if values is None else list(values) + [0.0] * idle
        self.ctx.fill(StepBatch(slots=slots, past_lens=past,
                                tokens=[[t] for t in tokens] + [[0]] * idle, rows=list(range(self.n_seqs)),
                                block_tables=cache.block_tables(slots), temperatures=pad(temperatures),
                                uniforms=pad(uniforms)))

    def _launch(self) -> None:
        eng, c = self.engine, self.ctx
        self.logits = eng.model.forward(c, eng.cache, c.rows)
        eng.lib.sample(self.logits, c.temperature, c.uniform, self.tokens_out)

    def run(self, slots, tokens, temperatures=None, uniforms=None) -> list:
        """The step for these sequences (at most as many as the graph was made for); returns their
        next tokens.  `logits`/`first_logits` hold a row per row of the graph, the live ones first."""
        eng = self.engine
        n = len(slots)
        if not 1 <= n <= self.n_seqs:
            raise ValueError(f"a captured step for {self.n_seqs} sequences cannot run {n}")
        q = [1] * n
        eng.cache.reserve(slots, q)
        self._fill(slots, tokens, temperatures, uniforms)
        if self.graph is None:
            # The first step for this batch size is launched kernel by kernel, on a side stream so
            # that allocations settle, and its result is the step's result; then the same launches
            # are captured for the steps after it.  Capturing executes nothing, so a mixer that
            # updates a state of its own has updated it once.
            side = torch.cuda.Stream(device=eng.device)
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                self._launch()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            out = self.tokens_out.tolist()[:n]
            first_logits = self.logits.clone()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                self._launch()
            self.graph = graph
            self.first_logits = first_logits
            eng.cache.commit(slots, q)
            return out
        self.first_logits = None
        self.graph.replay()
        out = self.tokens_out.tolist()[:n]
        eng.cache.commit(slots, q)
        return out
