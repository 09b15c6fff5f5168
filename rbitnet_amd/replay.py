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
