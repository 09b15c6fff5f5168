"""The product planners against every choice they could have made.

    python bench.py --planner-sweep [--model NAME ...] [--tokens 1,8,64,512,2048]

For the four products of a layer of each named shape (q/k/v, output, gate/up with the gated
epilogue, down) and each token count, the product is timed with the planner's own choice and
with every tile configuration and number of K slices forced in turn (more than 16 tokens), or
with every number of row tiles per wave and of waves, the token-resident variant on and off
(up to 16 tokens).  One line per product: the planner's time, the best forced time and which
choice that was.  W is rotated over copies that together exceed the caches, so that every
repetition reads it from memory as a step of a model does.
"""
from __future__ import annotations

import sys
from typing import Dict, List, Sequence, Tuple

TILE_CFGS = (4, 5, 6, 7, 8, 9, 10, 13)
SMALL_TILE_CFGS = (7, 10, 13)           # the tiles for at most 64 tokens


def products(cfg: Dict) -> List[Tuple[str, int, int, int]]:
    """(name, rows of W, K, epilogue) of a layer's four products."""
    e, f = cfg["hidden_size"], cfg["intermediate_size"]
    hq, hk = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    d = cfg.get("head_dim") or e // hq
    return [("qkv", (hq + 2 * hk) * d, e, 0), ("o", e, hq * d, 0), ("gate_up", 2 * f, e, 1), ("down", e, f, 0)]


def _time(lib, torch, fn, reps: int) -> float:
    fn(0)
    torch.cuda.synchronize()
    best = float("inf")
    for _ in range(3):
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for i in range(reps):
            fn(i)
        end.record()
        torch.cuda.synchronize()
        best = min(best, start.elapsed_time(end) * 1e3 / reps)
    return best


def sweep(models: Sequence[Tuple[str, Dict]], token_counts: Sequence[int], out=sys.stdout) -> float:
    """Prints the table; returns the worst ratio of the planner's time to the best forced time."""
    import torch
    from .csrc.lib import kernels
    from .errors import KernelError
    lib = kernels()
    L = lib._lib
    dev = torch.device("cuda:0")
    worst = 1.0
    print("| shape | product | rows x K | tokens | planner | us | best forced | us | planner / best |", file=out)
    print("|---|---|---|---|---|---|---|---|---|", file=out)
    for label, cfg in models:
        for name, n, k, epi in products(cfg):
            copies = max(2, min(8, (1 << 30) // (n * k * 2)))
            ws = [(torch.randn(n, k, device=dev) * 0.02).to(torch.bfloat16) for _ in range(copies)]
            for m in token_counts:
                a = (torch.randn(m, k, device=dev)).to(torch.bfloat16)
                c = torch.empty((m, n // 2 if epi else n), dtype=torch.bfloat16 if epi else torch.float32, device=dev)
                reps = max(4, min(40, int(2e4 / max(1.0, m * n * k * 2 / 1e9))))
                run = lambda i: lib.gemm_bf16(a, ws[i % copies], c, epi, w_frag=True)
                try:
                    L.rb_tune_tiles(0, 0)
                    L.rb_tune(0, 0)
                    L.rb_tune_use_resident(1)
                    L.rb_tune_use_stream(1)
                    plan = int(L.rb_tune_plan(m, n, k, epi))
                    chosen = f"tile {plan // 100} x {plan % 100}" if plan else "few-token kernels"
                    t_plan = _time(lib, torch, run, reps)
                    forced: List[Tuple[float, str]] = []
                    if m > 16:
                        for tile in (SMALL_TILE_CFGS if m <= 64 else TILE_CFGS):
                            if tile == 13 and k % 128:
                                continue
                            for parts in ((1,) if epi else ((1, 2, 4, 8) if m > 512 else range(1, 9))):
                                if (k // 64) % parts or k // 64 // parts < 4:
                                    continue
                                L.rb_tune_tiles(tile, parts)
                                try:
                                    forced.append((_time(lib, torch, run, reps), f"tile {tile} x {parts}"))
                                except KernelError:
                                    pass                    # a tile that does not take this many slices
                        L.rb_tune_tiles(0, 0)
                        if m <= 64:
                            L.rb_tune_use_stream(0)
                            forced.append((_time(lib, torch, run, reps), "few-token kernels"))
                            L.rb_tune_use_stream(1)
                    else:
                        for resident in (0, 2):
                            L.rb_tune_use_resident(resident)
                            if resident:
                                forced.append((_time(lib, torch, run, reps), "resident"))
                                continue
                            for r in (1, 2, 4):
                                if epi and r == 1:
                                    continue
                                for waves in (4, 8):
                                    L.rb_tune(r, waves)
                                    forced.append((_time(lib, torch, run, reps), f"skinny {r} tiles a wave, {waves} waves"))
                            L.rb_tune(0, 0)
                finally:
                    L.rb_tune_tiles(0, 0)
                    L.rb_tune(0, 0)
                    L.rb_tune_use_resident(1)
                    L.rb_tune_use_stream(1)
                t_best, which = min(forced)
                ratio = t_plan / t_best
                worst = max(worst, ratio)
                print(f"| {label} | {name} | {n} x {k} | {m} | {chosen} | {t_plan:.1f} | {which} | {t_best:.1f} | "
                      f"{ratio:.3f} |", file=out, flush=True)
            del ws
            torch.cuda.empty_cache()
    print(f"\nworst planner / best: {worst:.3f}", file=out)
    return worst
