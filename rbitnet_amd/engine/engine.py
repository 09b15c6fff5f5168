"""The engine: a model, its cache and ONE step function.

The reference's engine (crates/bitnet-core/src/inference.rs:74-209) owns one runtime
with one sequence and feeds it a token at a time (llama/runtime.rs:50-53,
llama/model.rs:219).  This one serves a batch of sequences that start together with
unequal lengths: `step` takes, per sequence, the tokens to run next (a whole prompt,
a piece of it, or one decoded token), runs exactly those as one packed batch on top of
what the cache holds, and returns float32 logits at the asked places only.

Guards as in model.rs:221-227: a token id outside the vocabulary and a position beyond
the model's or the cache's limit are errors raised before anything is launched.
"""
from __future__ import annotations

import sys
from collections import OrderedDict
from typing import Any, List, Optional, Sequence, Tuple, Union

import torch

from ..cache import PAGE_SIZE, Cache, pages_for
from ..cache.cache import bytes_per_token as cache_bytes_per_token
from ..config import load_config
from ..errors import CacheError, ConfigError, InferenceError
from ..weights import DEFAULT_SEED, RandomTensors, load_weights
from .context import StepBatch, StepContext, split_bucket
from .model import Model

DEFAULT_MAX_BATCH = 8
MAX_DECODE_GRAPHS = 24
CACHE_MEMORY_FRACTION = 0.9       # of the memory that is free after the weights, for a cache nobody sized
# A step's activations: the float32 stream, the projections before and after rotation, the gated
# product's input and output, partial sums of products cut along K.  About this many values of 4 bytes
# per token for every row of the widest matrix of a layer (measured at the 8B and 70B shapes: 3 to 4).
ACTIVATION_ROWS_PER_TOKEN = 4
STEP_TOKENS_SET_ASIDE = 8192      # a cache nobody sized leaves room for the activations of a step of this many tokens

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32,
           torch.bfloat16: torch.bfloat16, torch.float32: torch.float32}


def parse_dtype(dtype: Any) -> torch.dtype:
    if dtype not in _DTYPES:
        raise ConfigError(f"dtype must be 'bfloat16' or 'float32', found {dtype!r}")
    return _DTYPES[dtype]


class Engine:
    def __init__(self, config: Any, spec, model: Model, max_tokens: int, max_batch: int,
                 max_seq_len: Optional[int] = None):
        self.config = config
        self.spec = spec
        self.model = model
        self.lib = model.lib
        self.device = model.device
        self.dtype = model.dtype
        self.max_seq_len = min(int(max_seq_len or spec.max_positions), spec.max_positions)
        self.max_batch = int(max_batch)
        self.cache = Cache(model.cache_requests(), n_slots=self.max_batch, max_tokens=max_tokens,
                           dtype=self.dtype, device=self.device, readers=model.cache_readers())
        self.stats = {"steps": 0, "prefill_tokens": 0, "decode_tokens": 0}
        # per-kernel timers need every launch on its own
        self.use_graphs = bool(model.graph_safe) and getattr(self.lib, "times", None) is None
        # (rows of the captured step, split bucket) -> DecodeGraph, least recently used first
        self._graphs: "OrderedDict[Tuple[int, int], Any]" = OrderedDict()
        # steps other than the captured decode step: launches issued from C++ once a shape has been seen
        # before (step_plan.py); only for models whose parts do nothing on the device but call the library
        self.use_plans = bool(getattr(model, "plan_safe", False)) and getattr(self.lib, "times", None) is None
        from .step_plan import StepPlans
        self.plans = StepPlans(self)
        # float32 [sequences, vocab] of the last `decode_step`, valid until the next one
        self.last_decode_logits: Optional[torch.Tensor] = None
        from ..sampling import Sampler
        self.sampler = Sampler(self.lib, self.device)

    # ------------------------------------------------------------------ construction
    @classmethod
    def _build(cls, cfg: Any, spec, tensors_for, dtype: Any, max_tokens: Optional[int], max_batch: Optional[int],
               max_seq_len: Optional[int], device: str, generic_only: bool) -> "Engine":
        from ..csrc.lib import kernels
        lib = kernels()                       # raises when there is no GPU or no built library
        tdtype = parse_dtype(dtype)
        seq = min(int(max_seq_len or spec.max_positions), spec.max_positions)
        model = Model(spec, tdtype, device, lib, generic_only=generic_only, max_seq_len=seq)
        model.load(tensors_for(model, cfg))
        if max_batch is None:
            max_batch = DEFAULT_MAX_BATCH if max_tokens is None else max(1, min(pages_for(max_tokens), 1024))
        max_tokens = cls._cache_tokens(model, max_tokens, max_batch, seq)
        return cls(cfg, spec, model, max_tokens=max_tokens, max_batch=max_batch, max_seq_len=seq)

    @staticmethod
    def _cache_tokens(model: Model, max_tokens: Optional[int], max_batch: int, seq: int) -> int:
        """How many tokens the cache is made for.  Asked for: that many, or an error that says
        what fits.  Not asked for: every slot at the longest sequence, but no more than the memory
        that is free once the weights are placed (a message says so)."""
        per_token = cache_bytes_per_token(model.cache_requests(), model.dtype)
        fits = 1 << 40
        if per_token > 0 and model.device.type == "cuda":
            torch.cuda.empty_cache()          # what loading held for a moment counts as free
            free, _ = torch.cuda.mem_get_info(model.device)
            if max_tokens is None:            # nobody sized the cache: a step's activations keep their room
                free = max(0, free - model.activation_bytes(min(STEP_TOKENS_SET_ASIDE, max_batch * seq)))
            fits = int(free * CACHE_MEMORY_FRACTION) // per_token // PAGE_SIZE * PAGE_SIZE
        if max_tokens is not None:
            if pages_for(int(max_tokens)) * PAGE_SIZE > max(fits, PAGE_SIZE):
                raise CacheError(
                    f"a cache of max_tokens = {max_tokens} tokens ({per_token} bytes a token) does not fit the "
                    f"GPU's free memory; {fits} tokens would (lower max_tokens, or max_seq_len and max_batch)")
            return int(max_tokens)
        wanted = max_batch * pages_for(seq) * PAGE_SIZE
        if wanted > fits:
            print(f"[rbitnet_amd] cache: {max_batch} sequences of {seq} tokens would take "
                  f"{wanted * per_token / 2**30:.1f} GiB; sized to the {fits} tokens that fit free memory "
                  f"(give max_tokens or max_seq_len to choose)", file=sys.stderr, flush=True)
            if fits < PAGE_SIZE:
                raise CacheError("no memory is left for the cache once the weights are placed")
            return fits
        return wanted

    @classmethod
    def from_spec(cls, spec, tensors, dtype: Any = "bfloat16", max_tokens: int = 4096, max_batch: int = 8,
                  max_seq_len: Optional[int] = None, device: str = "cuda:0", generic_only: bool = False) -> "Engine":
        """An engine from a hand-made `ModelSpec` and tensors by name: what a new
        architecture's configuration class would produce, without one."""
        from ..csrc.lib import kernels
        model = Model(spec, parse_dtype(dtype), device, kernels(), generic_only=generic_only)
        model.load(tensors)
        return cls(None, spec, model, max_tokens=max_tokens, max_batch=max_batch, max_seq_len=max_seq_len)

    @classmethod
    def load_path(cls, path: str, dtype: Any = "bfloat16", max_tokens: Optional[int] = None,
                  max_batch: Optional[int] = None, max_seq_len: Optional[int] = None, device: str = "cuda:0",
                  generic_only: bool = False) -> "Engine":
        """A model folder (config.json + model.safetensors), as the reference's
        `Engine::load_path` takes a GGUF path (inference.rs:121-133)."""
        from ..weights.safetensors_io import WeightFolder
        cfg, spec = load_config(path, tensor_names=WeightFolder(path).names())

        def tensors_for(model: Model, cfg):
            aliases = getattr(type(cfg), "tensor_aliases", None)
            return load_weights(path, model.expected, aliases=aliases, ignored=spec.optional_tensors)

        return cls._build(cfg, spec, tensors_for, dtype, max_tokens, max_batch, max_seq_len, device, generic_only)

    @classmethod
    def random(cls, config: Any, seed: int = DEFAULT_SEED, dtype: Any = "bfloat16", std: float = 0.02,
               norm_std: float = 0.02, max_tokens: Optional[int] = None, max_batch: Optional[int] = None,
               max_seq_len: Optional[int] = None, device: str = "cuda:0", generic_only: bool = False) -> "Engine":
        """Random weights drawn on the GPU from a configuration and a seed, no files: the
        counterpart of the reference's toy mode (RBITNET_TOY / RBITNET_TOY_SEED,
        inference.rs:24-36).  The same model, bit for bit, as `write_random_model` with the
        same arguments writes (its stored dtype being this compute dtype)."""
        cfg, spec = load_config(config)

        def tensors_for(model: Model, cfg):
            store = torch.bfloat16 if model.dtype == torch.bfloat16 else torch.float32
            return RandomTensors(model.expected, seed, std, norm_std, store, device)

        return cls._build(cfg, spec, tensors_for, dtype, max_tokens, max_batch, max_seq_len, device, generic_only)

    # ------------------------------------------------------------------ slots
    def alloc_slot(self) -> int:
        return self.cache.alloc_slot()

    def free_slot(self, slot: int) -> None:
        self.cache.free_slot(slot)

    def length(self, slot: int) -> int:
        return self.cache.length(slot)

    def room(self, slot: int) -> int:
        """How many more tokens the sequence may hold (model and engine limits)."""
        return self.max_seq_len - self.cache.length(slot)

    # ------------------------------------------------------------------ the step
    def step(self, entries: Sequence[Tuple[int, Sequence[int]]],
             want: Union[str, Sequence[Sequence[int]]] = "last") -> torch.Tensor:
        """entries: (slot, tokens to run next) per sequence, at least one token each.
        want: "last" (the last token of each entry), "all", or per entry the indices
        among its tokens whose logits are asked for (may be empty).
        Returns float32 [number of asked places, vocab], in the order of entries and want."""
        if not entries:
            raise InferenceError("a step needs at least one sequence")
        slots = [int(s) for s, _ in entries]
        tokens = [list(t) for _, t in entries]
        vocab = self.spec.vocab_size
        past = []
        for s, toks in zip(slots, tokens):
            if not toks:
                raise InferenceError(f"slot {s}: a step brings at least one token per sequence")
            n = self.cache.length(s)
            if n + len(toks) > self.max_seq_len:
                raise InferenceError(
                    f"slot {s}: sequence position >= max_seq ({n} + {len(toks)} tokens exceed {self.max_seq_len})")
            for t in toks:
                if not 0 <= int(t) < vocab:
                    raise InferenceError(f"slot {s}: token id out of range ({t}, vocabulary {vocab})")
            past.append(n)
        rows: List[int] = []
        base = 0
        for i, toks in enumerate(tokens):
            if want == "last":
                idx = [len(toks) - 1]
            elif want == "all":
                idx = range(len(toks))
            else:
                idx = want[i]
            for j in idx:
                if not 0 <= int(j) < len(toks):
                    raise InferenceError(f"slot {slots[i]}: wanted place {j} is not among its {len(toks)} tokens")
                rows.append(base + int(j))
            base += len(toks)
        q_lens = [len(t) for t in tokens]
        if sum(q_lens) > 1024 and self.device.type == "cuda":
            # a long step's activations must fit beside the cache: say so before anything is reserved or launched
            need = self.model.activation_bytes(sum(q_lens), len(rows))
            free = torch.cuda.mem_get_info(self.device)[0] + torch.cuda.memory_reserved(self.device) \
                - torch.cuda.memory_allocated(self.device)
            if need > free:
                raise InferenceError(
                    f"a step of {sum(q_lens)} tokens needs about {need / 2**30:.1f} GiB for its activations and "
                    f"{free / 2**30:.1f} GiB are free: feed the prompts in pieces, or make the cache smaller")
        self.cache.reserve(slots, q_lens)
        batch = StepBatch(slots, past, tokens, rows, self.cache.block_tables(slots))
        logits = self.plans.run(batch) if self.use_plans else None
        if logits is None:
            ctx = StepContext.for_batch(self.device, batch, n_compute_units=self.lib.n_compute_units)
            logits = self.model.forward(ctx, self.cache, ctx.rows)
        self.cache.commit(slots, q_lens)
        self.stats["steps"] += 1
        if max(q_lens) == 1:
            self.stats["decode_tokens"] += len(slots)
        else:
            self.stats["prefill_tokens"] += sum(q_lens)
        return logits

    def decode_step(self, slots: Sequence[int], tokens: Sequence[int], temperatures=None, uniforms=None) -> list:
        """One token per sequence in, the next token per sequence out: a step and the
        sampling of its logits, replayed as a HIP graph (captured for a ladder of batch sizes, a
        batch running in the next size up with idle rows, see decode_graph.py);
        `use_graphs = False` runs the same kernels launch by launch."""
        slots = [int(s) for s in slots]
        tokens = [int(t) for t in tokens]
        vocab = self.spec.vocab_size
        for s, t in zip(slots, tokens):
            if not 0 <= t < vocab:
                raise InferenceError(f"slot {s}: token id out of range ({t}, vocabulary {vocab})")
            if self.cache.length(s) + 1 > self.max_seq_len:
                raise InferenceError(f"slot {s}: sequence position >= max_seq ({self.max_seq_len})")
        if not self.use_graphs:
            logits = self.step([(s, [t]) for s, t in zip(slots, tokens)], "last")
            self.last_decode_logits = logits
            return self.sampler.sample(logits, temperatures, uniforms)
        from .decode_graph import DecodeGraph, graph_size
        n = len(slots)
        key = (graph_size(n), split_bucket(max(self.cache.length(s) for s in slots) + 1))
        if key not in self._graphs:
            if len(self._graphs) >= MAX_DECODE_GRAPHS:
                self._graphs.popitem(last=False)           # the least recently used
            self._graphs[key] = DecodeGraph(self, key[0], key[1])
        self._graphs.move_to_end(key)
        graph = self._graphs[key]
        out = graph.run(slots, tokens, temperatures, uniforms)
        self.last_decode_logits = (graph.logits if graph.first_logits is None else graph.first_logits)[:n]
        self.stats["steps"] += 1
        self.stats["decode_tokens"] += n
        return out

    # ------------------------------------------------------------------ generation
    def generate(self, prompts: Sequence[Sequence[int]], max_tokens: Union[int, Sequence[int]] = 256, temperature: float = 0.7,
                 seed: int = 0, stop_token_ids: Optional[Sequence[int]] = None):
        from .generate import generate
        return generate(self, prompts, max_tokens=max_tokens, temperature=temperature, seed=seed,
                        stop_token_ids=stop_token_ids)

    def complete(self, prompt: Sequence[int], max_tokens: int = 256, temperature: float = 0.7, seed: int = 0):
        """One prompt in, its new tokens out: `Engine::complete(prompt, max_tokens,
        temperature)` of the reference (inference.rs:183) on token ids."""
        return self.generate([prompt], max_tokens=max_tokens, temperature=temperature, seed=seed)[0].tokens
