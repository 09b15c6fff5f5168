"""Decode and prefill throughput of the engine at the Llama-3-8B shape, one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B] [--no-points]
    rbitnet bench   (the same options)

A step is one decode step of the whole batch: the model's forward on one token per
sequence from the cache, and the choice of the next tokens on the GPU.  Weights are
random N(0, 0.02) bfloat16, token ids seeded uniform; prompts of 512 tokens are prefilled
first, so the timed steps run at contexts from 512 upwards (the reference publishes no
numbers, so `vs_baseline` is null).  One JSON line is printed.

  value               decoded tokens per second at the default batch (8)
  prefill             one prompt of 2,048 tokens: tokens/s, ms (the median of 5 runs after one
                      that warms up; min_ms beside it), fraction of the bf16 peak
  config.seq_len      the context the timed steps reach (prompt + warmup + steps + 1)
  roofline            bytes a decode step must read (weights once + live cache) / time
  points              decode tokens/s at batch 1 and 64
"""
from __future__ import annotations

import argparse
import json
import time

PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}
PEAK_HBM = 8.0e12

LLAMA3_8B = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 4096, "num_hidden_layers": 32,
    "num_attention_heads": 32, "num_key_value_heads": 8, "intermediate_size": 14336, "vocab_size": 128256,
    "rope_theta": 500000.0, "rms_norm_eps": 1e-5, "max_position_embeddings": 8192, "tie_word_embeddings": False,
}
# the other shapes the baseline names (configs[3] and [4]); chosen with --model
LLAMA2_7B = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 4096, "num_hidden_layers": 32,
    "num_attention_heads": 32, "num_key_value_heads": 32, "intermediate_size": 11008, "vocab_size": 32000,
    "rope_theta": 10000.0, "rms_norm_eps": 1e-5, "max_position_embeddings": 4096, "tie_word_embeddings": False,
}
LLAMA31_70B = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 8192, "num_hidden_layers": 80,
    "num_attention_heads": 64, "num_key_value_heads": 8, "intermediate_size": 28672, "vocab_size": 128256,
    "rope_theta": 500000.0, "rms_norm_eps": 1e-5, "max_position_embeddings": 8192, "tie_word_embeddings": False,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 8192},
}
# widths that no rule of the product planners was fitted to (measured as a check of those rules)
def _other(hidden, ff, heads, kv_heads, head_dim, layers, vocab=128256):
    return {"architectures": ["LlamaForCausalLM"], "hidden_size": hidden, "num_hidden_layers": layers,
            "num_attention_heads": heads, "num_key_value_heads": kv_heads, "head_dim": head_dim,
            "intermediate_size": ff, "vocab_size": vocab, "rope_theta": 500000.0, "rms_norm_eps": 1e-5,
            "max_position_embeddings": 8192, "tie_word_embeddings": False}


MODELS = {"llama3_8b": ("Llama-3-8B shape", LLAMA3_8B), "llama2_7b": ("Llama-2-7B shape", LLAMA2_7B),
          "llama31_70b": ("Llama-3.1-70B shape", LLAMA31_70B),
          "w2048": ("hidden 2048, 32 heads of 64 on 8", _other(2048, 8192, 32, 8, 64, 16)),
          "w3072": ("hidden 3072, 24 heads of 128 on 8", _other(3072, 8192, 24, 8, 128, 28)),
          "w5120": ("hidden 5120, 40 heads of 128 on 40", _other(5120, 13824, 40, 40, 128, 40, vocab=32000))}
PROMPT_LEN = 512
NEW_TOKENS = 256
PREFILL_TOKENS = 2048
PREFILL_RUNS = 5


def _sync():
    import torch
    torch.cuda.synchronize()


def matmul_flops_per_token(cfg) -> float:
    e, f, v = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    hq, hk = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    d = cfg.get("head_dim") or e // hq
    per_layer = 2 * (e * (hq + 2 * hk) * d + hq * d * e + 3 * e * f)
    return per_layer * cfg["num_hidden_layers"], 2 * e * v


def decode_run(engine, batch: int, steps: int, warmup: int, seed: int = 0, prompt_len=PROMPT_LEN):
    """Prefill `batch` prompts of `prompt_len` tokens (a pair (lo, hi): lengths drawn
    uniformly from lo..hi), then time `steps` decode steps."""
    import numpy as np
    rng = np.random.default_rng(seed)
    vocab = engine.spec.vocab_size
    slots = [engine.alloc_slot() for _ in range(batch)]
    if isinstance(prompt_len, tuple):
        lens = [int(n) for n in rng.integers(prompt_len[0], prompt_len[1] + 1, size=batch)]
    else:
        lens = [prompt_len] * batch
    prompts = [[int(t) for t in rng.integers(0, vocab, size=n)] for n in lens]
    # prompts go in groups so that a step's activations stay modest
    group = max(1, 8192 // max(lens))
    last = []
    for i in range(0, batch, group):
        logits = engine.step([(s, p) for s, p in zip(slots[i:i + group], prompts[i:i + group])], "last")
        last.extend(engine.sampler.sample(logits))
    tokens = last
    ctx0 = sum(lens) / batch
    for _ in range(warmup):
        tokens = engine.decode_step(slots, tokens)
    _sync()
    t0 = time.perf_counter()
    for _ in range(steps):
        tokens = engine.decode_step(slots, tokens)
    _sync()
    dt = time.perf_counter() - t0
    ctx_mean = ctx0 + warmup + (steps - 1) / 2.0 + 1
    for s in slots:
        engine.free_slot(s)
    return dt, ctx_mean


def generate_run(engine, n_requests: int, prompt_len: int, seed: int = 0, lo: int = 16, hi: int = 256) -> dict:
    """`Engine.generate` for n requests whose limits are drawn from lo..hi, so that the batch
    shrinks by a sequence every few steps: the loop's wall time for the decoding part (the prompts'
    step is timed by itself and taken off) against the sum of what its steps take as captured
    steps of a fixed batch of the same size, measured one size after the other."""
    import numpy as np
    from .engine.decode_graph import graph_size
    rng = np.random.default_rng(seed)
    vocab = engine.spec.vocab_size
    prompts = [[int(t) for t in rng.integers(0, vocab, size=prompt_len)] for _ in range(n_requests)]
    limits = [int(v) for v in rng.integers(lo, hi + 1, size=n_requests)]
    # the prompts' step alone (twice: the first run warms up)
    for _ in range(2):
        slots = [engine.alloc_slot() for _ in prompts]
        _sync()
        t0 = time.perf_counter()
        engine.step(list(zip(slots, prompts)), "last")
        _sync()
        t_prompt = time.perf_counter() - t0
        for s in slots:
            engine.free_slot(s)
    walls = []
    for _ in range(2):                      # the second run finds every size captured
        _sync()
        t0 = time.perf_counter()
        results = engine.generate(prompts, max_tokens=limits, temperature=0.0, stop_token_ids=[])
        _sync()
        walls.append(time.perf_counter() - t0)
    assert [len(r.tokens) for r in results] == limits
    # a step feeds the sequences that have not yet reached their limit: step j (from 1) runs those with limit > j
    sizes = [sum(1 for m in limits if m > j) for j in range(1, max(limits))]
    per_size = {}
    for b in sorted(set(graph_size(v) for v in sizes if v)):
        dt, _ = decode_run(engine, b, 24, 4, seed=100 + b, prompt_len=prompt_len)
        per_size[b] = dt / 24
    expected = sum(per_size[graph_size(v)] for v in sizes if v)
    decoded = sum(limits) - n_requests          # every request's first token comes from the prompts' step
    out = {"requests": n_requests, "prompt_len": prompt_len, "new_tokens": sum(limits), "steps": len(sizes),
           "prompt_step_ms": round(t_prompt * 1e3, 2)}
    for label, wall in (("first_run", walls[0]), ("second_run", walls[1])):
        loop = wall - t_prompt
        out[label] = {"wall_ms": round(wall * 1e3, 1), "decode_ms": round(loop * 1e3, 1),
                      "decode_tokens_per_s": round(decoded / loop, 1), "over_fixed_batches": round(loop / expected, 3)}
    out["fixed_batches_ms"] = round(expected * 1e3, 1)
    out["fixed_batch_tokens_per_s"] = {str(b): round(b / t, 1) for b, t in per_size.items()}
    return out


def short_prompts_run(engine, lengths, runs: int = 7) -> dict:
    """One prompt of each length, `runs` times: the step's wall time launched from Python and issued
    from C++ as a recorded step (the median of the runs after the one that records)."""
    import numpy as np
    rng = np.random.default_rng(5)
    out = {}
    for n in lengths:
        prompt = [int(t) for t in rng.integers(0, engine.spec.vocab_size, size=n)]
        row = {}
        for label, plans in (("python_ms", False), ("recorded_ms", True)):
            engine.use_plans = plans
            times = []
            for _ in range(runs + 2):
                slot = engine.alloc_slot()
                _sync()
                t0 = time.perf_counter()
                engine.step([(slot, prompt)], "last")
                _sync()
                times.append(time.perf_counter() - t0)
                engine.free_slot(slot)
            row[label] = round(sorted(times[2:])[runs // 2] * 1e3, 3)
        out[str(n)] = row
    engine.use_plans = True
    return out


def probe(lib, device) -> dict:
    """What this GPU reaches on a streaming read (`read_*`: all workgroups striding through the
    buffer together with plain loads; `stream_*`: every workgroup walking pieces of its own with
    non-temporal loads, as the decode products read their weights) and on back-to-back bfloat16 MFMAs
    (csrc/probe.hip): the practical ceilings beside the nominal peaks.  Timed with events on
    the stream, so that launch overhead on the host does not count."""
    import torch
    sink = torch.zeros(1, dtype=torch.float32, device=device)

    def timed(fn, reps: int) -> float:
        fn(0)
        _sync()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for i in range(reps):
            fn(i)
        end.record()
        _sync()
        return start.elapsed_time(end) * 1e-3 / reps

    out = {}
    pool = torch.empty((3 << 30) // 4, dtype=torch.int32, device=device).fill_(1)
    for label, nbytes, pieces in (("read_1gb_gbps", 1 << 30, False), ("read_32mb_gbps", 32 << 20, False),
                                  ("stream_1gb_gbps", 1 << 30, True), ("stream_32mb_gbps", 32 << 20, True)):
        copies = pool.numel() * 4 // nbytes
        views = [pool[i * (nbytes // 4):(i + 1) * (nbytes // 4)] for i in range(copies)]
        best = 0.0
        for blocks in (1024, 2048, 4096, 8192):          # the best grid size counts
            t = timed(lambda i: lib.probe_read(views[i % copies], sink, blocks, pieces),
                      12 if nbytes >= (1 << 30) else 96)
            best = max(best, nbytes / t)
        out[label] = round(best / 1e9, 1)
    del pool
    waves = 256 * 4 * 2
    t = timed(lambda i: lib.probe_mfma(waves, 20000, sink), 2)
    out["mfma_bf16_tflops"] = round(float(waves) * 20000 * 4 * 2 * 32 * 32 * 16 / t / 1e12, 1)
    return out


def load_probe(cfg, tokens: int, reps: int = 12) -> None:
    """For a profiler that counts cycles (`rocprofv3 --pmc GRBM_GUI_ACTIVE SQ_VALU_MFMA_BUSY_CYCLES --kernel-trace`):
    the MFMA probe, the gated product of the named shape with `tokens` tokens and the same product with 8 tokens,
    `reps` launches of each in a row.  GRBM_GUI_ACTIVE of a launch over its duration is the clock the GPU ran
    at, which under a product of many tokens is far below the one the nominal peak is quoted at."""
    import torch
    from .csrc.lib import kernels
    lib = kernels()
    dev, bf = "cuda:0", torch.bfloat16
    sink = torch.zeros(1 << 20, device=dev)
    for _ in range(reps):
        lib.probe_mfma(4096, 4000, sink)
    _sync()
    n, k = 2 * cfg["intermediate_size"], cfg["hidden_size"]
    w = torch.empty(n, k, device=dev, dtype=bf).normal_(0, 0.02)
    x = torch.randn(tokens, k, device=dev, dtype=bf)
    out = torch.empty(tokens, n // 2, device=dev, dtype=bf)
    for _ in range(reps):
        lib.gemm_bf16(x, w, out, 1, w_frag=False)
    _sync()
    wf = torch.empty_like(w)
    lib.place_rows(w, wf, frag=True)
    x8, o8 = x[:8].contiguous(), torch.empty(8, n // 2, device=dev, dtype=bf)
    for _ in range(reps):
        lib.gemm_bf16_few(x8, wf, o8, 1, w_frag=True)
    _sync()


def stream_probe(cfg, tokens: int = 8, copies: int = 8) -> dict:
    """The products of a decode step beside a kernel that only reads as many bytes (csrc/probe.hip, every
    workgroup walking pieces of its own with non-temporal loads, the best of four grid sizes): what a layer's
    products could reach at most if the arithmetic, the tokens and the epilogues cost nothing.  Both as a
    captured graph of `copies` launches over as many different matrices, so that W comes from memory."""
    import torch
    from .csrc.lib import kernels
    lib = kernels()
    dev, bf = "cuda:0", torch.bfloat16

    def per_launch(fn) -> float:
        for i in range(copies):
            fn(i)
        _sync()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for i in range(copies):
                fn(i)
        graph.replay()
        _sync()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(20):
            graph.replay()
        end.record()
        _sync()
        return start.elapsed_time(end) / 20 / copies * 1e3

    e, f, v = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    d = cfg.get("head_dim") or e // cfg["num_attention_heads"]
    qd, kd = cfg["num_attention_heads"] * d, cfg["num_key_value_heads"] * d
    sink = torch.zeros(1, device=dev)
    out = {}
    for name, n, k, kind in (("qkv", qd + 2 * kd, e, "prepared"), ("o_proj", e, qd, "to_stream"),
                             ("gate_up", 2 * f, e, "gated"), ("down", e, f, "to_stream"), ("output", v, e, "prepared")):
        ws = []
        for _ in range(copies):
            w = torch.empty(n, k, device=dev, dtype=bf).normal_(0, 0.02)
            wf = torch.empty_like(w)
            lib.place_rows(w, wf, frag=True)
            ws.append(wf)
            del w
        a = torch.randn(tokens, k, device=dev).to(bf)
        squares = torch.rand(tokens, (k + 15) // 16, device=dev) * 16
        if kind == "to_stream":
            c, gain = torch.zeros(tokens, n, device=dev), torch.ones(n, device=dev)
            gained, sq = torch.empty(tokens, n, dtype=bf, device=dev), torch.empty(tokens, (n + 15) // 16, device=dev)
            fn = lambda i: lib.gemm_bf16_few(a, ws[i], c, 3, gain=gain, gained=gained, squares_out=sq, w_frag=True)
        elif kind == "gated":
            c = torch.empty(tokens, n // 2, dtype=bf, device=dev)
            fn = lambda i: lib.gemm_bf16_few(a, ws[i], c, 1, squares=squares, eps=1e-5, w_frag=True)
        else:
            c = torch.empty(tokens, n, device=dev)
            fn = lambda i: lib.gemm_bf16_few(a, ws[i], c, 0, squares=squares, eps=1e-5, w_frag=True)
        product = per_launch(fn)
        views = [w.view(torch.int32) for w in ws]
        read = min(per_launch(lambda i: lib.probe_read(views[i], sink, blocks, True)) for blocks in (512, 1024, 2048, 4096))
        out[name] = {"mb": round(n * k * 2 / 1e6, 1), "product_us": round(product, 2), "read_us": round(read, 2)}
        del ws, views
    return out


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="bench")
    ap.add_argument("--gpus", type=int, default=1)
    # 16 + 240 steps: each sequence decodes the 256 tokens of the baseline's workload
    ap.add_argument("--steps", type=int, default=240)
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the configuration has")
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--dtype", default="bf16", choices=["bf16", "fp32"])
    ap.add_argument("--no-points", action="store_true", help="skip prefill and the batch 1 / 64 points")
    ap.add_argument("--points", default="1,64", help="batch sizes of the extra decode points")
    ap.add_argument("--model", default="llama3_8b",
                    help=f"shape to measure, one of {', '.join(sorted(MODELS))} (default: the baseline's configs[2]); "
                         "with --planner-sweep several, separated by commas")
    ap.add_argument("--planner-sweep", action="store_true",
                    help="no benchmark: time every product of the named shapes with the planner's choice and with "
                         "every choice forced (see planner_check.py)")
    ap.add_argument("--generate", type=int, default=0, metavar="N",
                    help="no benchmark line: Engine.generate for N requests with limits drawn from 16..256 against "
                         "captured steps of fixed batches (see generate_run)")
    ap.add_argument("--short-prompts", default="", metavar="N,N,...",
                    help="no benchmark line: one prompt of each of these lengths, launched from Python and issued "
                         "from C++ as a recorded step")
    ap.add_argument("--load-probe", action="store_true",
                    help="no benchmark line: a few launches in a row of the MFMA probe and of the named shape's gated "
                         "product with --prefill-tokens and with 8 tokens, for a profiler that counts cycles")
    ap.add_argument("--stream-probe", action="store_true",
                    help="no benchmark line: the named shape's decode products of 8 tokens beside a kernel that only "
                         "reads as many bytes")
    ap.add_argument("--tokens", default="1,8,64,512,2048", help="token counts of --planner-sweep")
    ap.add_argument("--sweep-detail", default=None, help="--planner-sweep: a file for every candidate's time")
    ap.add_argument("--prefill-tokens", type=int, default=PREFILL_TOKENS,
                    help="length of the one prompt whose prefill is timed")
    ap.add_argument("--prompt-len", default=str(PROMPT_LEN),
                    help="context at which decoding starts; LO,HI draws unequal lengths uniformly")
    args = ap.parse_args(argv)
    if args.gpus != 1:
        print(f"bench.py measures one GPU only (this library has no multi-GPU path); --gpus {args.gpus} is not run")
        return 2

    names = [v for v in args.model.split(",") if v]
    for name in names:
        if name not in MODELS:
            ap.error(f"unknown --model {name!r}; one of {', '.join(sorted(MODELS))}")
    if args.planner_sweep:
        from .planner_check import sweep
        detail = open(args.sweep_detail, "w") if args.sweep_detail else None
        sweep([(MODELS[n][0], MODELS[n][1]) for n in names], [int(v) for v in args.tokens.split(",") if v],
              detail=detail)
        return 0
    if len(names) != 1:
        ap.error("one --model at a time")
    if args.load_probe:
        load_probe(MODELS[names[0]][1], args.prefill_tokens)
        return 0
    if args.stream_probe:
        print(json.dumps(stream_probe(MODELS[names[0]][1])))
        return 0

    import torch
    from .engine import Engine

    if "," in args.prompt_len:
        lo, hi = (int(v) for v in args.prompt_len.split(","))
        prompt_len, longest = (lo, hi), hi
    else:
        prompt_len = longest = int(args.prompt_len)
    model_name, base = MODELS[args.model]
    cfg = dict(base)
    full_layers = cfg["num_hidden_layers"]
    if args.layers:
        cfg["num_hidden_layers"] = args.layers
    layers = cfg["num_hidden_layers"]
    dtype = "bfloat16" if args.dtype == "bf16" else "float32"
    max_batch = max([args.batch, args.generate] + ([] if args.no_points else [int(v) for v in args.points.split(",") if v]))
    ctx_cap = longest + max(NEW_TOKENS, args.steps + args.warmup) + 64
    prefill_tokens = args.prefill_tokens
    max_tokens = max(max_batch * ctx_cap, prefill_tokens + 64)
    max_seq_len = max(ctx_cap, prefill_tokens + 64)
    # contexts beyond what the named configuration allows are measured with its limit raised
    cfg["max_position_embeddings"] = max(cfg["max_position_embeddings"], max_seq_len)
    engine = Engine.random(cfg, seed=0, dtype=dtype, std=0.02, norm_std=0.0, max_batch=max_batch,
                           max_tokens=max_tokens, max_seq_len=max_seq_len)
    _sync()
    if args.generate:
        print(json.dumps(generate_run(engine, args.generate, longest)))
        return 0
    if args.short_prompts:
        print(json.dumps(short_prompts_run(engine, [int(v) for v in args.short_prompts.split(",") if v])))
        return 0

    dt, ctx_mean = decode_run(engine, args.batch, args.steps, args.warmup, prompt_len=prompt_len)
    ms = dt / args.steps * 1e3
    value = args.batch * args.steps / dt

    hk = cfg["num_key_value_heads"]
    d = cfg.get("head_dim") or cfg["hidden_size"] // cfg["num_attention_heads"]
    esize = 2 if args.dtype == "bf16" else 4
    kv_bytes_per_token = 2 * hk * d * esize * layers
    step_bytes = engine.model.weight_bytes() + args.batch * ctx_mean * kv_bytes_per_token
    achieved = step_bytes / (dt / args.steps)

    out = {
        "metric": f"decode tok/s at batch {args.batch} ({model_name})", "value": round(value, 2), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": args.dtype,
        "data": "synthetic: random N(0,0.02) weights, seeded uniform token ids",
        "config": {
            "model": model_name, "global_batch": args.batch, "seq_len": longest + args.warmup + args.steps + 1,
            "prompt_len": args.prompt_len if "," in args.prompt_len else longest, "parallelism": "single GPU", "layers": layers, "layers_full": full_layers,
            "hidden_size": cfg["hidden_size"], "heads": cfg["num_attention_heads"], "kv_heads": hk, "head_dim": d,
            "intermediate_size": cfg["intermediate_size"], "vocab_size": cfg["vocab_size"],
            "rope_theta": cfg["rope_theta"], "rms_norm_eps": cfg["rms_norm_eps"],
            "context": cfg["max_position_embeddings"], "mean_context": round(ctx_mean, 1),
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": PEAK_HBM / 1e9, "unit": "GB/s",
                     "frac": round(achieved / PEAK_HBM, 4)},
    }

    if not args.no_points:
        # ---- prefill of one prompt of 2,048 tokens
        import numpy as np
        rng = np.random.default_rng(1)
        prompt = [int(t) for t in rng.integers(0, cfg["vocab_size"], size=prefill_tokens)]
        times = []
        for i in range(PREFILL_RUNS + 1):
            slot = engine.alloc_slot()
            _sync()
            t0 = time.perf_counter()
            engine.step([(slot, prompt)], "last")
            _sync()
            times.append(time.perf_counter() - t0)
            engine.free_slot(slot)
        pt = sorted(times[1:])[len(times[1:]) // 2]           # the median; the first run warms up
        layer_flops, head_flops = matmul_flops_per_token(cfg)
        attn_flops = 4.0 * cfg["num_attention_heads"] * d * layers * (prefill_tokens * (prefill_tokens + 1) / 2.0)
        flops = layer_flops * prefill_tokens + head_flops * 1 + attn_flops
        out["prefill"] = {"value": round(prefill_tokens / pt, 1), "tokens": prefill_tokens, "ms": round(pt * 1e3, 3),
                          "frac": round(flops / pt / PEAK_FLOPS[args.dtype], 4), "runs": PREFILL_RUNS,
                          "min_ms": round(min(times[1:]) * 1e3, 3)}
        points, fracs = {}, {}
        for b in [int(v) for v in args.points.split(",") if v]:      # the same prompts and number of steps as the headline batch
            dtb, ctx_b = decode_run(engine, b, args.steps, args.warmup, seed=b, prompt_len=prompt_len)
            points[f"decode_b{b}"] = round(b * args.steps / dtb, 2)
            fracs[f"decode_b{b}"] = round((engine.model.weight_bytes() + b * ctx_b * kv_bytes_per_token)
                                          / (dtb / args.steps) / PEAK_HBM, 4)
        out["points"] = points
        out["points_roofline_frac"] = fracs      # as `roofline.frac`, for each point
        # the practical ceilings of this GPU, for reading the fractions above
        out["probe"] = probe(engine.lib, engine.device)

    print(json.dumps(out))
    return 0

