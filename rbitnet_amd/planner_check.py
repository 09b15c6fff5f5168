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


def _time_all(torch, candidates, run, reps: int, rounds: int = 5) -> List[float]:
    """The least time in microseconds of every candidate (a function that sets the choice up) over
    `rounds` rounds in which the candidates take turns, so that a drift of the clock or of the
    memory's state touches all of them alike; a candidate that the kernels refuse gets inf."""
    from .errors import KernelError
    best = [float("inf")] * len(candidates)
    alive = [True] * len(candidates)
    for _ in range(rounds):
        for j, setup in enumerate(candidates):
            if not alive[j]:
                continue
            setup()
            try:
                run(0)
            except KernelError:
                alive[j] = False
                continue
            start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            start.record()
            for i in range(reps):
                run(i + 1)
            end.record()
            torch.cuda.synchronize()
            best[j] = min(best[j], start.elapsed_time(end) * 1e3 / reps)
    return best


def sweep(models: Sequence[Tuple[str, Dict]], token_counts: Sequence[int], out=sys.stdout, detail=None) -> float:
    """Prints the table; returns the worst ratio of the planner's time to the best forced time.
    detail: a file that gets one line per product with the time of every candidate."""
    import torch
    from .csrc.lib import kernels
    lib = kernels()
    L = lib._lib
    dev = torch.device("cuda:0")
    worst = 1.0

    def reset():
        L.rb_tune_tiles(0, 0)
        L.rb_tune(0, 0)
        L.rb_tune_resident(0)
        L.rb_tune_use_resident(1)
        L.rb_tune_use_stream(1)

    def tile(cfg, parts):
        return lambda: (reset(), L.rb_tune_tiles(cfg, parts))

    def skinny(r, waves):
        return lambda: (reset(), L.rb_tune_use_resident(0), L.rb_tune(r, waves))

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
                reset()
                plan = int(L.rb_tune_plan(m, n, k, epi))
                chosen = f"tile {plan // 100} x {plan % 100}" if plan else "few-token kernels"
                names, setups = ["planner"], [reset]
                if m > 16:
                    for cfg_id in (SMALL_TILE_CFGS if m <= 64 else TILE_CFGS):
                        if cfg_id == 13 and k % 128:
                            continue
                        for parts in ((1,) if epi else ((1, 2, 4, 8) if m > 512 else range(1, 9))):
                            if (k // 64) % parts or k // 64 // parts < 4:
                                continue
                            names.append(f"tile {cfg_id} x {parts}")
                            setups.append(tile(cfg_id, parts))
                    if m <= 64:
                        names.append("few-token kernels")
                        setups.append(lambda: (reset(), L.rb_tune_use_stream(0)))
                else:
                    for tiles in (0, 1, 2, 4, 8):
                        names.append("resident" if tiles == 0 else f"resident, {tiles} row tiles a workgroup")
                        setups.append(lambda tiles=tiles: (reset(), L.rb_tune_use_resident(2), L.rb_tune_resident(tiles)))
                    for r in (1, 2, 4):
                        if epi and r == 1:
                            continue
                        for waves in (4, 8):
                            names.append(f"skinny {r} tiles a wave, {waves} waves")
                            setups.append(skinny(r, waves))
                try:
                    times = _time_all(torch, setups, run, reps)
                finally:
                    reset()
                t_plan = times[0]
                t_best, which = min(zip(times[1:], names[1:]))
                ratio = t_plan / t_best
                worst = max(worst, ratio)
                print(f"| {label} | {name} | {n} x {k} | {m} | {chosen} | {t_plan:.1f} | {which} | {t_best:.1f} | "
                      f"{ratio:.3f} |", file=out, flush=True)
                if detail is not None:
                    print(f"{label}; {name} {n} x {k}; {m} tokens; planner: {chosen}; " +
                          "; ".join(f"{nm}: {t:.1f}" for nm, t in zip(names, times)), file=detail, flush=True)
            del ws
            torch.cuda.empty_cache()
    print(f"\nworst planner / best: {worst:.3f}", file=out)
    return worst
