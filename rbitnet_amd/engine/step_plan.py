"""A step whose launches are issued from C++: recorded once, replayed when a step of the same
shape comes back.

A step of a 32-layer model is some three hundred launches; issued from Python they cost the host
15 us each, more than the GPU needs for a prompt of a few dozen tokens.  The launches of a step
depend on its shape alone (sequences, tokens, rows asked for, the longest piece, the width of the
page tables, the split bucket of decode attention); everything else they read from device buffers.
So a shape that has been seen before is recorded while it runs (the library notes every launch,
see csrc/plan.hip) and from then on replayed with one call.  What makes that sound:

* the step's device buffers are the same at every replay: the step layout (`StepContext`) belongs
  to the plan and is filled again before each replay, and every tensor the forward pass allocates
  comes from a memory pool of the plan's own, which nothing else allocates from;
* only parts whose forward does nothing on the device but call the kernel library can be
  replayed this way (`plan_safe`; a part that runs torch operations of its own is not: nobody
  would issue those again), and a model with any other part runs launch by launch as before;
* the logits are copied out of the pool before they are returned.

The decode step of generation has its own, faster form (a HIP graph, decode_graph.py); this one
serves every other step: prompts, prompts in pieces, steps of a replayed trace.
"""
from __future__ import annotations

import gc
import weakref
from collections import OrderedDict
from typing import Dict, Optional, Tuple

import torch

from .context import StepBatch, StepContext, split_bucket

MAX_PLANS = 16             # recorded shapes kept, least recently used first out
MAX_PLAN_TOKENS = 4096     # larger steps are bound by the GPU, and their buffers would be held for long
SEEN_KEYS = 256


def plan_key(batch: StepBatch) -> Tuple:
    q_lens = [len(t) for t in batch.tokens]
    widths = tuple(sorted((key, max(1, max(len(r) for r in table))) for key, table in batch.block_tables.items()))
    longest = max(p + q for p, q in zip(batch.past_lens, q_lens))
    return (len(q_lens), sum(q_lens), len(batch.rows), max(q_lens), widths, split_bucket(longest))


class StepPlan:
    def __init__(self, engine, key: Tuple):
        n_seqs, n_tokens, n_rows, _, widths, bucket = key
        # no cycle of references with the engine: a plan and its pool go when the engine goes, at once,
        # and not whenever the collector of cycles comes by
        self.engine = engine if isinstance(engine, weakref.ProxyType) else weakref.proxy(engine)
        self.ctx = StepContext(engine.device, n_seqs, n_tokens, n_rows, dict(widths), bucket=bucket,
                               n_compute_units=engine.lib.n_compute_units)
        self.pool = torch.cuda.MemPool()
        self.handle: Optional[int] = None
        self.logits: Optional[torch.Tensor] = None
        self.calls = 0

    def record(self, batch: StepBatch) -> torch.Tensor:
        """Runs the step launch by launch, noting the launches; the result is the step's result."""
        eng = self.engine
        self.ctx.fill(batch)
        self.handle = eng.lib.plan_begin()
        # While allocations go to this plan's pool no other pool may be destroyed (the allocator aborts):
        # the collector of cycles, which might find an old engine's plans, waits until the step is recorded.
        collecting = gc.isenabled()
        gc.disable()
        try:
            with torch.cuda.use_mem_pool(self.pool, device=eng.device):
                self.logits = eng.model.forward(self.ctx, eng.cache, self.ctx.rows)
        except BaseException:
            eng.lib.plan_free(self.handle)
            self.handle = None
            raise
        finally:
            if collecting:
                gc.enable()
        self.calls = eng.lib.plan_end(self.handle)
        return self.logits.clone()

    def replay(self, batch: StepBatch) -> torch.Tensor:
        self.ctx.fill(batch)
        self.engine.lib.plan_replay(self.handle)
        return self.logits.clone()

    def close(self) -> None:
        if self.handle is not None:
            try:
                self.engine.lib.plan_free(self.handle)
            except ReferenceError:            # the engine is gone already; the library outlives it
                from ..csrc.lib import kernels
                kernels().plan_free(self.handle)
            self.handle = None
        self.logits = None
        self.pool = None

    def __del__(self) -> None:
        try:
            self.close()
        except Exception:
            pass


class StepPlans:
    """The recorded steps of an engine.  A shape is recorded the second time it is seen (most shapes
    of a varied load never come back, and a recording holds its buffers), and at most MAX_PLANS are kept."""

    def __init__(self, engine):
        self.engine = weakref.proxy(engine)
        self.plans: "OrderedDict[Tuple, StepPlan]" = OrderedDict()
        self.seen: "OrderedDict[Tuple, int]" = OrderedDict()
        self.stats: Dict[str, int] = {"recorded": 0, "replayed": 0}

    def run(self, batch: StepBatch) -> Optional[torch.Tensor]:
        """The step's logits through a plan, or None when this step is to be run the ordinary way."""
        if sum(len(t) for t in batch.tokens) > MAX_PLAN_TOKENS:
            return None
        key = plan_key(batch)
        plan = self.plans.get(key)
        if plan is not None:
            self.plans.move_to_end(key)
            self.stats["replayed"] += 1
            return plan.replay(batch)
        if key not in self.seen:
            self.seen[key] = 1
            if len(self.seen) > SEEN_KEYS:
                self.seen.popitem(last=False)
            return None
        if len(self.plans) >= MAX_PLANS:
            _, old = self.plans.popitem(last=False)
            old.close()
        plan = StepPlan(self.engine, key)
        try:
            logits = plan.record(batch)
        except torch.cuda.OutOfMemoryError:
            # no room to hold a step's buffers: give back what the plans hold and go on without them
            plan.close()
            self.clear()
            self.engine.use_plans = False
            torch.cuda.empty_cache()
            return None
        self.plans[key] = plan
        self.stats["recorded"] += 1
        return logits

    def clear(self) -> None:
        for plan in self.plans.values():
            plan.close()
        self.plans.clear()
