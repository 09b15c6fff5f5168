"""The generation loop above the step function.

Reference, one sequence (crates/bitnet-core/src/llama/runtime.rs:34-78): run the
prompt, then up to max_tokens times: sample; if the token is a stop token, end without
emitting it or feeding it (:67-69); else emit it and run it (:70-72).  An empty prompt
has nothing to run (:46-48); here it is an error unless a BOS id is configured.

Here the same runs for batches: all prompts of a batch in one step, then one token per
sequence still running.  A sequence that ends gives its slot back at once and the rest
go on; when a batch is done the next one starts in the same slots, until every request
has been served.  Results are independent of what else was in the batch.  Unlike
runtime.rs:71 no step is run whose logits nobody reads: a sequence that has reached
max_tokens does not feed its last token.

`engine` needs: alloc_slot(), free_slot(slot), step(entries, want) -> logits,
sampler.sample(logits, temperatures, uniforms) -> tokens, decode_step(slots, tokens,
temperatures, uniforms) -> tokens, max_batch, max_seq_len,
cache.n_pages / cache.kv_groups (for admission), spec.stop_token_ids.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional, Sequence

from ..cache.pages import pages_for
from ..errors import InferenceError
from ..sampling.sampler import uniform


@dataclass
class GenerationResult:
    tokens: List[int] = field(default_factory=list)
    finish_reason: str = ""          # "stop" | "length" | "context"
    prompt_tokens: int = 0


@dataclass
class _Running:
    index: int                       # position of the request in the caller's list
    slot: int
    budget: int                      # new tokens it may still emit
    room: int                        # tokens the sequence may still hold
    result: GenerationResult = None


def decide(token: int, emitted: int, max_tokens: int, room_after: int, stop_ids) -> Optional[str]:
    """What a freshly sampled token means for its sequence.  None: emit it and go on.
    "stop": a stop token, not emitted.  "length": emitted, and it was the last one
    allowed.  "context": emitted, but the sequence cannot hold another token."""
    if token in stop_ids:
        return "stop"
    if emitted + 1 >= max_tokens:
        return "length"
    if room_after <= 0:
        return "context"
    return None


def plan_batches(prompt_lens: Sequence[int], max_tokens: int, max_batch: int, max_seq_len: int,
                 page_budget: int) -> List[List[int]]:
    """Requests in order, cut into batches that fit the slots and the pages: a request
    counts with the most tokens it can come to hold."""
    batches: List[List[int]] = []
    cur: List[int] = []
    used = 0
    for i, n in enumerate(prompt_lens):
        need = pages_for(min(n + max_tokens, max_seq_len))
        if need > page_budget:
            need = page_budget            # it will end with "context" when the pages run out
        if cur and (len(cur) >= max_batch or used + need > page_budget):
            batches.append(cur)
            cur, used = [], 0
        cur.append(i)
        used += need
    if cur:
        batches.append(cur)
    return batches


def generate(engine, prompts: Sequence[Sequence[int]], max_tokens: int = 256, temperature: float = 0.7,
             seed: int = 0, stop_token_ids: Optional[Sequence[int]] = None) -> List[GenerationResult]:
    """Defaults as the reference's request fields: max_tokens 256, temperature 0.7
    (crates/bitnet-server/src/lib.rs:317, :358)."""
    stop_ids = set(engine.spec.stop_token_ids) | set(int(t) for t in (stop_token_ids or ()))
    bos = getattr(engine.spec, "bos_token_id", None)
    prompts = [list(p) for p in prompts]
    for i, p in enumerate(prompts):
        if not p:
            if bos is None:
                raise InferenceError(f"request {i}: empty prompt (and the model names no BOS token)")
            prompts[i] = [int(bos)]
        if len(prompts[i]) > engine.max_seq_len:
            raise InferenceError(f"request {i}: prompt of {len(prompts[i])} tokens exceeds max_seq {engine.max_seq_len}")
    results = [GenerationResult(prompt_tokens=len(p)) for p in prompts]
    if max_tokens <= 0:
        for r in results:
            r.finish_reason = "length"
        return results
    page_budget = min((g.table.pool.n for g in engine.cache.kv_groups), default=1 << 30)
    for i, p in enumerate(prompts):
        if pages_for(len(p)) > page_budget:
            raise InferenceError(f"request {i}: prompt of {len(p)} tokens does not fit the cache")
    batches = plan_batches([len(p) for p in prompts], max_tokens, engine.max_batch, engine.max_seq_len, page_budget)

    for batch in batches:
        running: List[_Running] = []
        for i in batch:
            slot = engine.alloc_slot()
            running.append(_Running(index=i, slot=slot, budget=max_tokens,
                                    room=engine.max_seq_len - len(prompts[i]), result=results[i]))
        try:
            logits = engine.step([(r.slot, prompts[r.index]) for r in running], "last")
            tokens = engine.sampler.sample(
                logits, [temperature] * len(running),
                [uniform(seed, r.index, 0) for r in running] if temperature > 0 else None)
            while running:
                survivors: List[_Running] = []
                feed: List[int] = []
                for r, tok in zip(running, tokens):
                    verdict = decide(tok, len(r.result.tokens), max_tokens, r.room - 1, stop_ids)
                    if verdict != "stop":
                        r.result.tokens.append(int(tok))
                        r.room -= 1
                    # a sequence that cannot get another page ends here as well
                    if verdict is None and not _has_page_for(engine, r.slot):
                        verdict = "context"
                    if verdict is None:
                        survivors.append(r)
                        feed.append(int(tok))
                    else:
                        r.result.finish_reason = verdict
                        engine.free_slot(r.slot)
                        r.slot = -1
                running = survivors
                if running:
                    tokens = engine.decode_step(
                        [r.slot for r in running], feed, [temperature] * len(running),
                        [uniform(seed, r.index, len(r.result.tokens)) for r in running] if temperature > 0 else None)
        finally:
            for r in running:
                if r.slot >= 0:
                    engine.free_slot(r.slot)
    return results


def _has_page_for(engine, slot: int) -> bool:
    """Whether one more token fits the sequence's pages or a free page is left."""
    n = engine.cache.length(slot)
    for g in engine.cache.kv_groups:
        if pages_for(n + 1) > len(g.table.pages(slot)) and g.table.pool.n_free == 0:
            return False
    return True
