"""The `rbitnet` command line, in the manner of the reference's (`rbitnet <subcommand>`,
crates/rbitnet-cli/src/main.rs:14-97; options fall back to RBITNET_* environment
variables as its `#[arg(long, env = ...)]` do; failures print `error: ...` and exit
with 1, main.rs:300-303).

    rbitnet generate --model DIR --prompt-ids 1,2,3 [--prompt-ids 4,5 ...] [--max-tokens 256]
                     [--temperature 0.7] [--seed 0] [--stop-token-ids 2,7] [--add-bos] [--dtype bfloat16]
    rbitnet random   --config config.json --out DIR [--seed 42] [--init-std 0.02] [--norm-std 0.02]
    rbitnet inspect  DIR_OR_FILE
    rbitnet replay   --model DIR --dtype D --out DIR --max-tokens N   < trace.jsonl        (steps)
    rbitnet replay   --model DIR --dtype D --out DIR --max-tokens N --requests FILE --mode whole|tail|batched
                     [--batch-size B]                                                     (whole requests)
    rbitnet bench    [--steps K] [--warmup W] [--batch B] [--layers L] [--no-points]

Environment, as the reference's engine reads it (crates/bitnet-core/src/inference.rs:16-41):
RBITNET_MODEL (default of --model; must not contain '..', inference.rs:44-53), RBITNET_TOY=1
(random weights instead of a weight file: needs --config) with RBITNET_TOY_SEED (default 42),
RBITNET_MAX_TOKENS_CAP (ceiling of --max-tokens, default 8192,
crates/bitnet-server/src/config.rs:42).  The library works on token ids: there is no
tokenizer, and no `serve` or `models` subcommand.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
from typing import List, Optional

from .errors import ConfigError, RbitnetError


def _truthy(name: str) -> bool:
    return os.environ.get(name, "") in ("1", "true", "yes")        # inference.rs:16-29


def _no_parent_components(path: str) -> str:
    if ".." in path.replace("\\", "/").split("/"):
        raise ConfigError("path must not contain '..' components")
    return path


def _ids(text: str) -> List[int]:
    try:
        return [int(t) for t in text.replace(" ", ",").split(",") if t != ""]
    except ValueError:
        raise ConfigError(f"token ids must be integers separated by commas, found {text!r}") from None


def _cache_need(prompt_lens: List[int], max_tokens: int, max_batch: int, limit: int):
    """What the request asks of the cache: the longest sequence it can come to, and the most
    tokens that `max_batch` prompts in a row can come to hold together (each rounded up to the
    cache's unit of 64 tokens)."""
    most = [min(n + max_tokens, limit) for n in prompt_lens]
    rounded = [(n + 63) // 64 * 64 for n in most]
    together = max(sum(rounded[i:i + max_batch]) for i in range(0, max(1, len(rounded) - max_batch + 1)))
    return max(most), together


def _engine(args, prompt_lens: List[int], max_tokens: int):
    from .config import load_config
    from .engine import Engine
    model = args.model or os.environ.get("RBITNET_MODEL")
    if os.environ.get("RBITNET_MODEL") and not args.model:
        _no_parent_components(model)
    toy = _truthy("RBITNET_TOY") or getattr(args, "random", False)
    config = (getattr(args, "config", None) or model) if toy else model
    if not config:
        raise ConfigError("random weights need --config (a config.json or a folder holding one)" if toy else
                          "model not loaded; pass --model DIR or set RBITNET_MODEL (or RBITNET_TOY=1 with --config)")
    # the cache is made for this request, not for the longest context the configuration allows
    _, spec = load_config(config)
    limit = min(args.max_seq_len or spec.max_positions, spec.max_positions)
    longest, together = _cache_need(prompt_lens, max_tokens, args.max_batch, limit)
    kw = dict(dtype=args.dtype, max_batch=args.max_batch, max_seq_len=args.max_seq_len or longest,
              max_tokens=together)
    if toy:
        seed = args.weight_seed if args.weight_seed is not None else int(os.environ.get("RBITNET_TOY_SEED", "42"))
        cfg_path = os.path.join(config, "config.json") if os.path.isdir(config) else config
        with open(cfg_path) as f:
            return Engine.random(json.load(f), seed=seed, **kw)
    return Engine.load_path(model, **kw)


def cmd_generate(args) -> int:
    cap = int(os.environ.get("RBITNET_MAX_TOKENS_CAP", "8192"))
    if args.max_tokens > cap:
        raise ConfigError(f"max_tokens exceeds cap ({args.max_tokens}, max {cap})")
    prompts = [_ids(p) for p in (args.prompt_ids or [])]
    if args.prompt_file:
        with open(args.prompt_file) as f:
            for line in f:
                line = line.strip()
                if not line:
                    continue
                prompts.append(json.loads(line) if line.startswith("[") else _ids(line))
    if not prompts:
        raise ConfigError("no prompt given (--prompt-ids or --prompt-file)")
    engine = _engine(args, [len(p) + 1 for p in prompts], args.max_tokens)
    if args.add_bos:
        bos = engine.spec.bos_token_id
        if bos is None:
            raise ConfigError("--add-bos: the model's configuration names no BOS token (bos_token_id)")
        prompts = [[int(bos)] + p for p in prompts]
    stop = _ids(args.stop_token_ids) if args.stop_token_ids else None
    results = engine.generate(prompts, max_tokens=args.max_tokens, temperature=args.temperature, seed=args.seed,
                              stop_token_ids=stop)
    for p, r in zip(prompts, results):
        print(json.dumps({"prompt_tokens": len(p), "tokens": r.tokens, "finish_reason": r.finish_reason}))
    return 0


def cmd_random(args) -> int:
    import torch
    from .weights import write_random_model
    dtype = {"bfloat16": torch.bfloat16, "float32": torch.float32}[args.dtype]
    seed = args.seed if args.seed is not None else int(os.environ.get("RBITNET_TOY_SEED", "42"))
    folder = write_random_model(args.out, args.config, seed=seed, std=args.init_std, norm_std=args.norm_std,
                                dtype=dtype)
    print(f"wrote {folder}")
    return 0


def cmd_inspect(args) -> int:
    """Summary line, configuration, first 20 tensors and "... and N more", as the
    reference's inspect_gguf prints them (crates/bitnet-core/examples/inspect_gguf.rs:22-50)."""
    from .weights.safetensors_io import WeightFolder
    path = args.path
    store = WeightFolder(path)
    names = store.names()
    n_bytes = sum(f.data_len for f in store.files)
    arch = "?"
    folder = path if os.path.isdir(path) else os.path.dirname(path)
    cfg_path = os.path.join(folder, "config.json")
    raw = None
    if os.path.isfile(cfg_path):
        with open(cfg_path) as f:
            raw = json.load(f)
        arch = (raw.get("architectures") or ["?"])[0]
    print(f"safetensors arch={arch} tensors={len(names)} files={len(store.files)}")
    print(f"tensor_data_len={n_bytes} bytes")
    if raw is not None:
        from .config import load_config
        cfg, spec = load_config(raw)
        fields = {k: v for k, v in vars(cfg).items() if not k.startswith("_")}
        print(f"{type(cfg).__name__}: " + " ".join(f"{k}={v!r}" for k, v in fields.items()))
        from .engine.model import expected_tensors
        from .weights.loader import resolve_names
        expected = expected_tensors(spec)
        _, missing, unexpected = resolve_names(expected, names, getattr(type(cfg), "tensor_aliases", None),
                                               ["lm_head.weight"] if spec.head_name is None else [])
        print(f"expected tensors={len(expected)} missing={len(missing)} unexpected={len(unexpected)}")
    show = min(20, len(names))
    print(f"First {show} tensors:")
    for n in names[:show]:
        dtype, shape = store.info(n)
        print(f"  {n:50} dims={list(shape)} dtype={dtype}")
    if len(names) > show:
        print(f"  ... and {len(names) - show} more")
    return 0


def cmd_replay(args) -> int:
    from .engine import Engine
    from .replay import replay
    if args.requests:
        from .replay import replay_requests
        with open(args.requests) as f:
            requests = [json.loads(line) for line in f if line.strip()]
        engine = Engine.load_path(args.model, dtype=args.dtype, max_tokens=args.max_tokens,
                                  max_batch=max(1, args.batch_size))
        replay_requests(engine, requests, args.mode, args.out, batch_size=args.batch_size)
        return 0
    engine = Engine.load_path(args.model, dtype=args.dtype, max_tokens=args.max_tokens)
    replay(engine, sys.stdin, args.out)
    return 0


def cmd_bench(args) -> int:
    from .benchmark import main as bench_main
    return bench_main(args.rest)


def build_parser() -> argparse.ArgumentParser:
    ap = argparse.ArgumentParser(prog="rbitnet", description="rbitnet_amd: Llama-decoder generation on one MI355X")
    sub = ap.add_subparsers(dest="command", required=True)

    g = sub.add_parser("generate", help="generate token ids from prompts of token ids")
    g.add_argument("--model", help="folder with config.json and model.safetensors [env: RBITNET_MODEL]")
    g.add_argument("--config", help="config.json for random weights (with --random or RBITNET_TOY=1)")
    g.add_argument("--random", action="store_true", help="random weights instead of a weight file")
    g.add_argument("--weight-seed", type=int, default=None, help="seed of random weights [env: RBITNET_TOY_SEED, 42]")
    g.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    g.add_argument("--prompt-ids", action="append", help="comma-separated token ids (repeatable)")
    g.add_argument("--prompt-file", help="file with one prompt a line (comma-separated ids or a JSON list)")
    g.add_argument("--max-tokens", type=int, default=256)
    g.add_argument("--temperature", type=float, default=0.7)
    g.add_argument("--seed", type=int, default=0, help="seed of the sampler")
    g.add_argument("--stop-token-ids", help="comma-separated ids that end a sequence (besides the model's EOS)")
    g.add_argument("--add-bos", action="store_true", help="put the model's BOS token before every prompt")
    g.add_argument("--max-batch", type=int, default=8, help="sequences that run together")
    g.add_argument("--max-seq-len", type=int, default=None, help="most tokens a sequence may hold")
    g.set_defaults(fn=cmd_generate)

    r = sub.add_parser("random", help="write a model folder with random weights")
    r.add_argument("--config", required=True)
    r.add_argument("--out", required=True)
    r.add_argument("--seed", type=int, default=None, help="[env: RBITNET_TOY_SEED, 42]")
    r.add_argument("--init-std", type=float, default=0.02)
    r.add_argument("--norm-std", type=float, default=0.02)
    r.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    r.set_defaults(fn=cmd_random)

    i = sub.add_parser("inspect", help="print what a model folder or safetensors file holds")
    i.add_argument("path")
    i.set_defaults(fn=cmd_inspect)

    p = sub.add_parser("replay", help="replay a trace of token ids from standard input and write logits")
    p.add_argument("--model", required=True)
    p.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    p.add_argument("--out", required=True)
    p.add_argument("--max-tokens", type=int, required=True)
    p.add_argument("--requests", help="a file of whole requests, one JSON object a line: {\"id\": .., \"tokens\": [..]}; "
                                      "without it, steps are read from standard input")
    p.add_argument("--mode", default="whole", choices=["whole", "tail", "batched"],
                   help="how --requests are cut into steps (the logits must not depend on it)")
    p.add_argument("--batch-size", type=int, default=4, help="requests that run together in --mode batched")
    p.set_defaults(fn=cmd_replay)

    b = sub.add_parser("bench", help="decode and prefill throughput at the Llama-3-8B shape (one JSON line)",
                       add_help=False)
    b.add_argument("rest", nargs=argparse.REMAINDER)
    b.set_defaults(fn=cmd_bench)
    return ap


def main(argv: Optional[List[str]] = None) -> int:
    argv = list(sys.argv[1:] if argv is None else argv)
    if argv and argv[0] == "bench":             # its options are the benchmark's own
        from .benchmark import main as bench_main
        return bench_main(argv[1:])
    args = build_parser().parse_args(argv)
    try:
        return args.fn(args)
    except RbitnetError as e:
        print(f"error: {e}", file=sys.stderr)
        return 1
    except BrokenPipeError:
        # the reader of our output has gone (`... | head`): not an error of ours; point stdout at
        # /dev/null so that the interpreter's flush at exit does not complain either
        os.dup2(os.open(os.devnull, os.O_WRONLY), sys.stdout.fileno())
        return 0
    except OSError as e:
        print(f"error: IO error: {e}", file=sys.stderr)
        return 1


if __name__ == "__main__":
    sys.exit(main())
