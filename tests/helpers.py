"""Tiny configurations, model folders and oracle logits shared by the tests."""
from __future__ import annotations

import os
import tempfile
from functools import lru_cache

import numpy as np
import torch

# Two tiny Llama configurations that differ in every size and option, and a third whose
# sizes let the bfloat16 path take its matrix-core kernels (head size 64, widths that are
# multiples of 16, head_dim given explicitly and not hidden / heads).
TINY_A = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 64, "num_hidden_layers": 2,
    "num_attention_heads": 4, "num_key_value_heads": 2, "intermediate_size": 172, "vocab_size": 256,
    "rope_theta": 10000.0, "rms_norm_eps": 1e-5, "max_position_embeddings": 128,
    "tie_word_embeddings": False, "rope_style": "interleaved",      # the reference's pairing; B has none: "half"
}
TINY_B = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 96, "num_hidden_layers": 3,
    "num_attention_heads": 4, "num_key_value_heads": 1, "intermediate_size": 256, "vocab_size": 384,
    "rope_theta": 500000.0, "rms_norm_eps": 1e-6, "max_position_embeddings": 256,
    "rope_scaling": {"rope_type": "llama3", "factor": 8.0, "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                     "original_max_position_embeddings": 32},
    "tie_word_embeddings": True, "eos_token_id": 7,
}
TINY_C = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 192, "num_hidden_layers": 2,
    "num_attention_heads": 8, "num_key_value_heads": 2, "head_dim": 64, "intermediate_size": 336,
    "vocab_size": 500, "rope_theta": 10000.0, "rms_norm_eps": 1e-5, "max_position_embeddings": 512,
    "tie_word_embeddings": False, "rope_style": "half",
}
# one layer with room for a thousand positions, for what only long contexts show
TINY_D = {
    "architectures": ["LlamaForCausalLM"], "hidden_size": 128, "num_hidden_layers": 1,
    "num_attention_heads": 4, "num_key_value_heads": 1, "head_dim": 64, "intermediate_size": 208,
    "vocab_size": 300, "rope_theta": 10000.0, "rms_norm_eps": 1e-5, "max_position_embeddings": 1088,
    "tie_word_embeddings": True,
}
CONFIGS = {"A": (TINY_A, 0, 0.02), "B": (TINY_B, 1, 0.0), "C": (TINY_C, 2, 0.02), "D": (TINY_D, 3, 0.02)}

_FOLDERS = {}
_TMP = None


def model_folder(name: str) -> str:
    """A model folder with random bfloat16 weights for the named tiny configuration,
    written once per test session into a temporary directory."""
    global _TMP
    if name not in _FOLDERS:
        import rbitnet_amd
        if _TMP is None:
            _TMP = tempfile.TemporaryDirectory(prefix="rbitnet_models_")
        cfg, seed, norm_std = CONFIGS[name]
        folder = os.path.join(_TMP.name, name)
        # std 0.1 rather than 0.02: with tiny widths, larger weights make attention and the
        # gate matter, so that a wrong pairing or mask shows in the logits
        rbitnet_amd.write_random_model(folder, cfg, seed=seed, std=0.1, norm_std=norm_std, dtype=torch.bfloat16)
        _FOLDERS[name] = folder
    return _FOLDERS[name]


def tokens_for(name: str, length: int, seed: int) -> list:
    vocab = CONFIGS[name][0]["vocab_size"]
    rng = np.random.default_rng(1000 * seed + length)
    return [int(t) for t in rng.integers(0, vocab, size=length)]


@lru_cache(maxsize=None)
def _plain(name: str):
    from plain_llama import PlainLlama
    return PlainLlama.from_folder(model_folder(name))


@lru_cache(maxsize=None)
def plain_logits(name: str, tokens: tuple) -> torch.Tensor:
    """float64 logits [T, V] of the plain implementation (cached per sequence)."""
    return _plain(name).logits(list(tokens))


@lru_cache(maxsize=None)
def _plain_rounded(name: str):
    from plain_llama import PlainLlama
    return PlainLlama.from_folder(model_folder(name), round_bf16=True)


@lru_cache(maxsize=None)
def plain_logits_rounded(name: str, tokens: tuple) -> torch.Tensor:
    """The plain implementation rounding to bfloat16 where an engine that computes in bfloat16
    stores values in that type: what such an engine can come close to."""
    return _plain_rounded(name).logits(list(tokens))


def max_err(got: torch.Tensor, want: torch.Tensor) -> float:
    """Largest absolute difference relative to the largest wanted magnitude."""
    want = want.to(torch.float64)
    got = got.detach().to("cpu", torch.float64)
    return float((got - want).abs().max() / want.abs().max().clamp_min(1e-30))


# error bounds relative to the largest logit: float32 differs from the float64 oracle by
# summation order and float32 rounding only; bfloat16 rounds activations to 8 bits of
# mantissa at each layer boundary
TOL = {"float32": 2e-5, "bfloat16": 3e-2}
# The bfloat16 engine against the plain implementation that rounds where the engine stores
# bfloat16.  The two cannot agree value by value: a difference far below one rounding step before
# a value is rounded becomes a whole step with the matching probability, so after a few roundings
# in a row two computations that round at the same places are as far from each other as each is
# from the exact result.  What they share is the size of that distance: its root mean square over
# a request's logits is a stable number (the engine's is 0.93 to 1.05 of the plain one's over sixty
# requests of four models; 0.84 to 1.13 over the 8 x V logits of steps of single tokens), so a
# systematic error of a thousandth of the largest logit already shows.
BF16_RMS_RATIO = 1.15          # a step of many tokens
BF16_RMS_RATIO_FEW = 1.3       # 8 single-token steps (fewer logits, folded norms)
BF16_MAX_RATIO = 1.5           # the largest error against the plain one's largest


def rms_err(got: torch.Tensor, want: torch.Tensor) -> float:
    """Root mean square difference relative to the largest wanted magnitude."""
    want = want.to(torch.float64)
    got = got.detach().to("cpu", torch.float64)
    return float(((got - want) ** 2).mean().sqrt() / want.abs().max().clamp_min(1e-30))


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor, block: int = 16) -> torch.Tensor:
    """Blocks of 16 gate rows, each followed by the 16 up rows of the same columns: the layout
    the gated product's epilogue reads, built here with torch as the oracle of the packing kernel."""
    ff, k = gate.shape
    g = gate.reshape(ff // block, block, k)
    u = up.reshape(ff // block, block, k)
    return torch.stack([g, u], dim=1).reshape(2 * ff, k).contiguous()


def fragment_major(w: torch.Tensor) -> torch.Tensor:
    """[N, K] (N % 16 == 0, K % 32 == 0) in the matrix-core products' other layout of W: blocks of
    16 rows x 32 columns in the order [N / 16][K / 32]; inside a block the value of row r, column q
    at 8 * (16 * (q / 8) + r) + q % 8.  Built with torch, as the oracle of the packing kernel."""
    n, k = w.shape
    return w.reshape(n // 16, 16, k // 32, 4, 8).permute(0, 2, 3, 1, 4).contiguous().view(n, k)
