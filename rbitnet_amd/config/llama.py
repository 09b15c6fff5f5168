"""Typed configuration of the Llama dense decoder, read from config.json.

The reference reads the same ten numbers from GGUF metadata
(crates/bitnet-core/src/llama/config.rs:8-19, from_gguf :40-122); required keys,
defaults and checks follow it:

* required: width, layer count, head count, feed-forward width, vocabulary
  (config.rs:44-55, 74-92); a missing key is an error that names the key;
* defaults: kv heads = heads (:56), rope_theta 10000 (:94-97), rms_norm_eps
  1e-5 (:99-102), context 2048 (:104-107; the reference's cap of 8192 is a
  safety limit of its CPU engine and is not kept);
* checks: heads and kv heads positive and divisible (:57-61), width divisible by
  heads unless head_dim is given (:62-67), head_dim even (:68-72).

Keys are the ones a Llama config.json holds (hidden_size, num_hidden_layers,
...); the GGUF spellings the reference reads (llama.embedding_length, ...) are
accepted as alternates.  Not in the reference and accepted here: `head_dim`,
`rope_scaling` (llama3 rule), `tie_word_embeddings`, `eos_token_id`,
`bos_token_id`, and `rope_style`: which two numbers of a head the rotation pairs.
"interleaved" pairs (2i, 2i+1), as the reference's rope_inplace does
(model.rs:122-136): that fits weight files whose q and k rows were permuted for it
when they were exported, which the GGUF files that the reference reads are.  "half"
pairs (i, i + D/2): that fits weights stored under the names of a config.json's own
folder (`model.layers.N.self_attn.q_proj.weight`), which are not permuted.  Without
the key the tensor names decide (`with_tensor_names`): GGUF spellings (`blk.N.attn_q`)
give "interleaved", everything else, and a model without a weight file, "half".
"""
from __future__ import annotations

import json
import math
import os
import dataclasses
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from ..errors import ConfigError
from .spec import LayerSpec, ModelSpec, PartSpec

_MISSING = object()

# config.json key -> the GGUF metadata key the reference reads for the same number
_ALIASES = {
    "hidden_size": "llama.embedding_length",
    "num_hidden_layers": "llama.block_count",
    "num_attention_heads": "llama.attention.head_count",
    "num_key_value_heads": "llama.attention.head_count_kv",
    "intermediate_size": "llama.feed_forward_length",
    "vocab_size": "llama.vocab_size",
    "rope_theta": "llama.rope.freq_base",
    "rms_norm_eps": "llama.attention.layer_norm_rms_epsilon",
    "max_position_embeddings": "llama.context_length",
}


def _lookup(d: Dict[str, Any], key: str) -> Any:
    if key in d and d[key] is not None:
        return d[key]
    alias = _ALIASES.get(key)
    if alias and alias in d and d[alias] is not None:
        return d[alias]
    return _MISSING


def _as_int(name: str, value: Any) -> int:
    """JSON ints, or floats with an integral value (config.rs:21-29 accepts
    every integer width); negative numbers and everything else are errors."""
    if isinstance(value, bool):
        raise ConfigError(f"{name} must be an integer, found {value!r}")
    if isinstance(value, int):
        out = value
    elif isinstance(value, float) and value.is_integer():
        out = int(value)
    else:
        raise ConfigError(f"{name} must be an integer, found {value!r}")
    if out < 0:
        raise ConfigError(f"{name} must not be negative, found {out}")
    return out


def _as_float(name: str, value: Any) -> float:
    if isinstance(value, bool) or not isinstance(value, (int, float)):
        raise ConfigError(f"{name} must be a number, found {value!r}")
    out = float(value)
    if not math.isfinite(out):
        raise ConfigError(f"{name} must be finite, found {value!r}")
    return out


def _required_int(d: Dict[str, Any], key: str) -> int:
    v = _lookup(d, key)
    if v is _MISSING:
        raise ConfigError(f"missing {key}")
    return _as_int(key, v)


@dataclass
class RopeScaling:
    """The llama3 rule: wavelengths below original/high_freq_factor keep their
    frequency, above original/low_freq_factor it is divided by `factor`, and in
    between the two are blended linearly."""
    rope_type: str
    factor: float
    low_freq_factor: float
    high_freq_factor: float
    original_max_position_embeddings: int

    def as_dict(self) -> Dict[str, Any]:
        return {
            "rope_type": self.rope_type,
            "factor": self.factor,
            "low_freq_factor": self.low_freq_factor,
            "high_freq_factor": self.high_freq_factor,
            "original_max_position_embeddings": self.original_max_position_embeddings,
        }


def _parse_rope_scaling(value: Any) -> Optional[RopeScaling]:
    if value is None:
        return None
    if not isinstance(value, dict):
        raise ConfigError(f"rope_scaling must be an object or null, found {value!r}")
    kind = value.get("rope_type", value.get("type", "default"))
    if kind == "default":
        return None
    if kind != "llama3":
        raise ConfigError(f"unsupported rope_scaling rope_type {kind!r} (supported: 'default', 'llama3')")
    out = {}
    for key in ("factor", "low_freq_factor", "high_freq_factor"):
        if key not in value:
            raise ConfigError(f"missing rope_scaling.{key}")
        out[key] = _as_float(f"rope_scaling.{key}", value[key])
        if out[key] <= 0:
            raise ConfigError(f"rope_scaling.{key} must be positive, found {out[key]}")
    if "original_max_position_embeddings" not in value:
        raise ConfigError("missing rope_scaling.original_max_position_embeddings")
    orig = _as_int("rope_scaling.original_max_position_embeddings", value["original_max_position_embeddings"])
    if orig <= 0:
        raise ConfigError("rope_scaling.original_max_position_embeddings must be positive")
    if not out["high_freq_factor"] > out["low_freq_factor"]:
        raise ConfigError("rope_scaling.high_freq_factor must be greater than low_freq_factor")
    return RopeScaling("llama3", out["factor"], out["low_freq_factor"], out["high_freq_factor"], orig)


@dataclass
class LlamaConfig:
    hidden_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    rope_theta: float = 10000.0
    rope_scaling: Optional[RopeScaling] = None
    rope_style: Optional[str] = None      # None: not said; `effective_rope_style` decides
    rms_norm_eps: float = 1e-5
    max_position_embeddings: int = 2048
    tie_word_embeddings: bool = False
    eos_token_ids: List[int] = field(default_factory=list)
    bos_token_id: Optional[int] = None
    torch_dtype: Optional[str] = None

    architecture = "LlamaForCausalLM"

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "LlamaConfig":
        hidden = _required_int(d, "hidden_size")
        layers = _required_int(d, "num_hidden_layers")
        heads = _required_int(d, "num_attention_heads")
        kv = _lookup(d, "num_key_value_heads")
        kv_heads = heads if kv is _MISSING else _as_int("num_key_value_heads", kv)
        if heads == 0 or kv_heads == 0 or heads % kv_heads != 0:
            raise ConfigError(
                f"invalid num_attention_heads / num_key_value_heads: {heads} / {kv_heads} "
                "(both positive, heads a multiple of kv heads)")
        hd = _lookup(d, "head_dim")
        if hd is _MISSING:
            if hidden % heads != 0:
                raise ConfigError(f"hidden_size {hidden} not divisible by num_attention_heads {heads}")
            head_dim = hidden // heads
        else:
            head_dim = _as_int("head_dim", hd)
        if head_dim == 0 or head_dim % 2 != 0:
            raise ConfigError(f"invalid head_dim {head_dim}: must be even and positive")
        ff = _required_int(d, "intermediate_size")
        vocab = _required_int(d, "vocab_size")
        for name, val in (("hidden_size", hidden), ("num_hidden_layers", layers),
                          ("intermediate_size", ff), ("vocab_size", vocab)):
            if val == 0:
                raise ConfigError(f"{name} must be positive")

        theta = _lookup(d, "rope_theta")
        theta = 10000.0 if theta is _MISSING else _as_float("rope_theta", theta)
        if theta <= 0:
            raise ConfigError(f"rope_theta must be positive, found {theta}")
        eps = _lookup(d, "rms_norm_eps")
        eps = 1e-5 if eps is _MISSING else _as_float("rms_norm_eps", eps)
        if eps < 0:
            raise ConfigError(f"rms_norm_eps must not be negative, found {eps}")
        ctx = _lookup(d, "max_position_embeddings")
        ctx = 2048 if ctx is _MISSING else _as_int("max_position_embeddings", ctx)
        if ctx == 0:
            raise ConfigError("max_position_embeddings must be positive")

        act = d.get("hidden_act", "silu")
        if act != "silu":
            raise ConfigError(f"unsupported hidden_act {act!r} (supported: 'silu')")
        for key in ("attention_bias", "mlp_bias"):
            if d.get(key):
                raise ConfigError(f"{key}=true is not supported: the Llama dense decoder has no biases")
        style = d.get("rope_style")
        if style is not None and style not in ("interleaved", "half"):
            raise ConfigError(f"unsupported rope_style {style!r} (supported: 'interleaved', 'half')")

        eos = d.get("eos_token_id")
        if eos is None:
            eos_ids: List[int] = []
        elif isinstance(eos, list):
            eos_ids = [_as_int("eos_token_id", e) for e in eos]
        else:
            eos_ids = [_as_int("eos_token_id", eos)]
        bos = d.get("bos_token_id")
        bos_id = None if bos is None else _as_int("bos_token_id", bos)
        dt = d.get("torch_dtype", d.get("dtype"))

        return cls(
            hidden_size=hidden, num_hidden_layers=layers, num_attention_heads=heads,
            num_key_value_heads=kv_heads, head_dim=head_dim, intermediate_size=ff, vocab_size=vocab,
            rope_theta=theta, rope_scaling=_parse_rope_scaling(d.get("rope_scaling")), rope_style=style,
            rms_norm_eps=eps, max_position_embeddings=ctx,
            tie_word_embeddings=bool(d.get("tie_word_embeddings", False)),
            eos_token_ids=eos_ids, bos_token_id=bos_id, torch_dtype=dt if isinstance(dt, str) else None)

    @classmethod
    def from_file(cls, path: str) -> "LlamaConfig":
        if os.path.isdir(path):
            path = os.path.join(path, "config.json")
        with open(path) as f:
            return cls.from_dict(json.load(f))

    def to_dict(self) -> Dict[str, Any]:
        out: Dict[str, Any] = {
            "architectures": [self.architecture],
            "model_type": "llama",
            "hidden_size": self.hidden_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size,
            "vocab_size": self.vocab_size,
            "hidden_act": "silu",
            "rope_theta": self.rope_theta,
            "rope_scaling": self.rope_scaling.as_dict() if self.rope_scaling else None,
            "rms_norm_eps": self.rms_norm_eps,
            "max_position_embeddings": self.max_position_embeddings,
            "tie_word_embeddings": self.tie_word_embeddings,
        }
        if self.rope_style is not None:
            out["rope_style"] = self.rope_style
        if self.eos_token_ids:
            out["eos_token_id"] = self.eos_token_ids if len(self.eos_token_ids) > 1 else self.eos_token_ids[0]
        if self.bos_token_id is not None:
            out["bos_token_id"] = self.bos_token_id
        if self.torch_dtype:
            out["torch_dtype"] = self.torch_dtype
        return out

    # ------------------------------------------------------------------ pairing of the rotation
    def with_tensor_names(self, names) -> "LlamaConfig":
        """The configuration for a weight file that holds tensors of these names: where
        config.json does not say how the rotation pairs a head's numbers, files with the GGUF
        spellings (exported with q and k rows permuted for adjacent pairs) get "interleaved"."""
        if self.rope_style is None and any(n.startswith("blk.") or n.startswith("token_embd") for n in names):
            return dataclasses.replace(self, rope_style="interleaved")
        return self

    @property
    def effective_rope_style(self) -> str:
        return self.rope_style or "half"

    # ------------------------------------------------------------------ the spec
    def to_spec(self) -> ModelSpec:
        """The decoder of model.rs:229-315 as data: embedding, L pre-norm blocks
        of (RMSNorm, attention with rotary positions, RMSNorm, SiLU-gated
        feed-forward), final RMSNorm, output matrix."""
        position = PartSpec("rope", {
            "head_dim": self.head_dim,
            "theta": self.rope_theta,
            "scaling": self.rope_scaling.as_dict() if self.rope_scaling else None,
            "style": self.effective_rope_style,
            "max_positions": self.max_position_embeddings,
        })
        norm = PartSpec("rmsnorm", {"size": self.hidden_size, "eps": self.rms_norm_eps})
        layers = []
        for i in range(self.num_hidden_layers):
            mixer = PartSpec("attention", {
                "num_heads": self.num_attention_heads,
                "num_kv_heads": self.num_key_value_heads,
                "head_dim": self.head_dim,
                "scale": 1.0 / math.sqrt(self.head_dim),     # model.rs:260
                "window": None,
                "position": position,
                "cache_from": None,
                "names": {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight",
                          "o": "o_proj.weight"},
            })
            ffn = PartSpec("swiglu", {
                "intermediate_size": self.intermediate_size, "activation": "silu",
                "names": {"gate": "gate_proj.weight", "up": "up_proj.weight", "down": "down_proj.weight"}})
            layers.append(LayerSpec(prefix=f"model.layers.{i}", block="prenorm", mixer=mixer,
                                    feed_forward=ffn, norm1=norm, norm2=norm,
                                    segments={"norm1": "input_layernorm", "mixer": "self_attn",
                                              "norm2": "post_attention_layernorm", "feed_forward": "mlp"}))
        return ModelSpec(
            architecture=self.architecture,
            hidden_size=self.hidden_size,
            vocab_size=self.vocab_size,
            max_positions=self.max_position_embeddings,
            embedding_name="model.embed_tokens.weight",
            layers=layers,
            final_norm=norm,
            final_norm_name="model.norm.weight",
            head_name=None if self.tie_word_embeddings else "lm_head.weight",
            stop_token_ids=list(self.eos_token_ids),
            bos_token_id=self.bos_token_id,
            # an output matrix stored beside tied embeddings is not read
            optional_tensors=["lm_head.weight"] if self.tie_word_embeddings else [],
        )

    # the names a GGUF export of the same model uses (model.rs:146-179), accepted
    # by the loader as alternates of the names above
    @staticmethod
    def tensor_aliases(name: str) -> List[str]:
        table = {
            "model.embed_tokens.weight": ["embed_tokens.weight", "token_embd.weight", "token_embd"],
            "model.norm.weight": ["norm.weight", "output_norm.weight"],
            "lm_head.weight": ["output.weight"],
        }
        if name in table:
            return table[name]
        parts = name.split(".")
        if len(parts) >= 4 and parts[0] == "model" and parts[1] == "layers":
            n = parts[2]
            rest = ".".join(parts[3:])
            gguf = {
                "input_layernorm.weight": ["attn_norm.weight"],
                "self_attn.q_proj.weight": ["attn_q.weight"],
                "self_attn.k_proj.weight": ["attn_k.weight"],
                "self_attn.v_proj.weight": ["attn_v.weight"],
                "self_attn.o_proj.weight": ["attn_output.weight", "attn_out.weight"],
                "post_attention_layernorm.weight": ["ffn_norm.weight"],
                "mlp.gate_proj.weight": ["ffn_gate.weight"],
                "mlp.up_proj.weight": ["ffn_up.weight"],
                "mlp.down_proj.weight": ["ffn_down.weight"],
            }.get(rest, [])
            return [f"layers.{n}.{rest}"] + [f"blk.{n}.{g}" for g in gguf]
        return []
