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
temperatures, uniforms) -> tokens, max_batch, max_seq_len, spec.stop_token_ids and, for
admission, cache.token_capacity(), cache.tokens_needed(n) and cache.can_grow(slot): the
loop counts tokens and leaves to the cache how it stores them.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Callable, List, Optional, Sequence, Union

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
    budget: int                      # new tokens it may emit in all
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


def plan_batches(prompt_lens: Sequence[int], max_tokens, max_batch: int, max_seq_len: int,
                 capacity: int, needed: Callable[[int], int] = lambda n: n) -> List[List[int]]:
    """Requests in order, cut into batches that fit the slots and the cache: a request counts
    with the most tokens it can come to hold (max_tokens: one number, or one per request),
    `needed(n)` being what n tokens take of the cache's `capacity`."""
    batches: List[List[int]] = []
    cur: List[int] = []
    used = 0
    for i, n in enumerate(prompt_lens):
        new = max_tokens if isinstance(max_tokens, int) else max_tokens[i]
        need = needed(min(n + max(0, int(new)), max_seq_len))
        if need > capacity:
            need = capacity               # it will end with "context" when the cache is full
        if cur and (len(cur) >= max_batch or used + need > capacity):
            batches.append(cur)
            cur, used = [], 0
        cur.append(i)
        used += need
    if cur:
        batches.append(cur)
    return batches


def generate(engine, prompts: Sequence[Sequence[int]], max_tokens: Union[int, Sequence[int]] = 256,
             temperature: float = 0.7, seed: int = 0,
             stop_token_ids: Optional[Sequence[int]] = None) -> List[GenerationResult]:
    """Defaults as the reference's request fields: max_tokens 256, temperature 0.7
    (crates/bitnet-server/src/lib.rs:317, :358).  max_tokens may be one number per request, as
    every request of the reference carries its own."""
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
    if isinstance(max_tokens, int):
        limits = [int(max_tokens)] * len(prompts)
    else:
        limits = [int(m) for m in max_tokens]
        if len(limits) != len(prompts):
            raise InferenceError(f"{len(limits)} values of max_tokens for {len(prompts)} requests")
    order = [i for i in range(len(prompts)) if limits[i] > 0]
    for i in range(len(prompts)):
        if limits[i] <= 0:
            results[i].finish_reason = "length"
    if not order:
        return results
    cache = engine.cache
    capacity = cache.token_capacity()
    for i, p in enumerate(prompts):
        if cache.tokens_needed(len(p)) > capacity:
            raise InferenceError(f"request {i}: prompt of {len(p)} tokens does not fit the cache")
    batches = plan_batches([len(prompts[i]) for i in order], [limits[i] for i in order], engine.max_batch,
                           engine.max_seq_len, capacity, cache.tokens_needed)

    for batch in batches:
        running: List[_Running] = []
        for i in (order[j] for j in batch):
            slot = engine.alloc_slot()
            running.append(_Running(index=i, slot=slot, budget=limits[i],
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
                    verdict = decide(tok, len(r.result.tokens), r.budget, r.room - 1, stop_ids)
                    if verdict != "stop":
                        r.result.tokens.append(int(tok))
                        r.room -= 1
                    # a sequence that the cache cannot let grow ends here as well
                    if verdict is None and not cache.can_grow(r.slot):
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
