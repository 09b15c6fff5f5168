"""Trace replay: feeds given token ids through the engine step by step and writes the
logits.  It samples nothing and has no forward pass, cache or loader of its own: it
drives `Engine.load_path`, `alloc_slot`, `step` and `free_slot`, the ones generation
uses.

Input, one JSON object a line:
    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}
For a step in which something is wanted, `<out>/<step>.f32` holds the logits at the
wanted places in the order of the entries and of `want`, little-endian float32
[wanted, vocab].  After every step a line `done <step>` is printed and flushed.

The reference has no such tool; its closest relative is the planned export of golden
logits (docs/GOLDEN_TESTS.md:9-15).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
from typing import Dict, IO, Optional


from .errors import RbitnetError


def replay(engine, lines: IO[str], out_dir: str, log: IO[str] = sys.stdout) -> int:
    """Runs every step of `lines`; returns the number of steps."""
    os.makedirs(out_dir, exist_ok=True)
    slots: Dict[str, int] = {}
    n = 0
    for line in lines:
        line = line.strip()
        if not line:
            continue
        try:
            rec = json.loads(line)
        except json.JSONDecodeError as e:
            raise RbitnetError(f"trace line {n + 1} is not valid JSON: {e}") from None
        step = rec.get("step", n)
        entries = rec.get("entries", [])
        feed, want = [], []
        for e in entries:
            rid = str(e["id"])
            if rid not in slots:
                slots[rid] = engine.alloc_slot()
            feed.append((slots[rid], [int(t) for t in e["tokens"]]))
            want.append([int(w) for w in e.get("want", [])])
        if feed:
            logits = engine.step(feed, want)
            if logits.shape[0] > 0:
                arr = logits.detach().to("cpu").numpy().astype("<f4", copy=False)
                tmp = os.path.join(out_dir, f".{step}.f32.tmp")
                arr.tofile(tmp)
                os.replace(tmp, os.path.join(out_dir, f"{step}.f32"))
        for rid in rec.get("end", []):
            rid = str(rid)
            if rid not in slots:
                raise RbitnetError(f"step {step}: request {rid!r} ends but never started")
            engine.free_slot(slots.pop(rid))
        n += 1
        print(f"done {step}", file=log, flush=True)
    return n


def replay_requests(engine, requests, mode: str, out_dir: str, batch_size: int = 1, tail: int = 32) -> Dict[str, str]:
    """Whole requests instead of steps: `requests` is a list of {"id", "tokens"[, "prefill"]}; every
    request's logits at all its positions go to `<out>/<id>.npy` (float32 [T, vocab]) and an
    `index.json` names them.  The mode says how the tokens are cut into steps, which must not
    change the logits beyond rounding:
      whole    each request alone, all tokens in one step;
      tail     each request alone, all but the last `tail` tokens in one step, the rest one by one;
      batched  `batch_size` requests at a time in file order: their first tokens (all but the last
               `tail`, or the request's own "prefill" count) in one step of unequal lengths, then one
               token per request still running; a request that has run out leaves and frees its
               slot, and the next group starts in the same slots."""
    import numpy as np
    import torch
    if mode not in ("whole", "tail", "batched"):
        raise RbitnetError(f"unknown replay mode {mode!r} (whole, tail, batched)")
    os.makedirs(out_dir, exist_ok=True)
    reqs = [(str(r["id"]), [int(t) for t in r["tokens"]], r.get("prefill")) for r in requests]
    for rid, toks, _ in reqs:
        if not toks:
            raise RbitnetError(f"request {rid!r} has no tokens")
    index: Dict[str, str] = {}
    group = max(1, int(batch_size)) if mode == "batched" else 1
    for g0 in range(0, len(reqs), group):
        batch = reqs[g0:g0 + group]
        slots = [engine.alloc_slot() for _ in batch]
        heads = []
        for _, toks, prefill in batch:
            if mode == "whole":
                heads.append(len(toks))
            elif prefill is not None and mode == "batched":
                heads.append(max(1, min(int(prefill), len(toks))))
            else:
                heads.append(max(1, len(toks) - tail) if len(toks) > tail else 1)
        rows = [[] for _ in batch]
        logits = engine.step([(s, toks[:h]) for s, (_, toks, _), h in zip(slots, batch, heads)], "all")
        off = 0
        for i, h in enumerate(heads):
            rows[i].append(logits[off:off + h].to("cpu"))
            off += h
        done = list(heads)
        live = [i for i in range(len(batch)) if done[i] < len(batch[i][1])]
        for i in range(len(batch)):
            if i not in live:
                engine.free_slot(slots[i])
        while live:
            logits = engine.step([(slots[i], [batch[i][1][done[i]]]) for i in live], "last").to("cpu")
            for row, i in enumerate(live):
                rows[i].append(logits[row:row + 1])
                done[i] += 1
            for i in [i for i in live if done[i] >= len(batch[i][1])]:
                engine.free_slot(slots[i])
            live = [i for i in live if done[i] < len(batch[i][1])]
        for i, (rid, toks, _) in enumerate(batch):
            name = f"{rid}.npy"
            np.save(os.path.join(out_dir, name), torch.cat(rows[i]).numpy().astype("<f4", copy=False))
            index[rid] = name
    with open(os.path.join(out_dir, "index.json"), "w") as f:
        json.dump({"mode": mode, "requests": index}, f, indent=1)
    return index


def main(argv: Optional[list] = None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description="Replay a trace of token ids and write logits.")
    ap.add_argument("--model", required=True, help="folder with config.json and model.safetensors")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to 64); sizes the cache")
    args = ap.parse_args(argv)
    try:
        from .engine import Engine
        engine = Engine.load_path(args.model, dtype=args.dtype, max_tokens=args.max_tokens)
        replay(engine, sys.stdin, args.out)
    except RbitnetError as e:
        print(f"error: {e}", file=sys.stderr)
        return 1
    return 0


if __name__ == "__main__":
    sys.exit(main())
