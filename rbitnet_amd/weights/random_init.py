"""Random weights from a configuration and a seed, as a model folder or in memory.

The reference's counterpart is its toy model, filled from a seeded generator
(crates/bitnet-core/src/model/toy.rs:16-30, seed from RBITNET_TOY_SEED with
default 42, inference.rs:31-36).  Here every tensor the model's parts declare is
drawn by name: matrices N(0, std), norm gains 1 + N(0, norm_std).  Each tensor
has a generator of its own, seeded from (seed, name), so its values do not
depend on the order of the tensors or on which others exist.
"""
from __future__ import annotations

import hashlib
import json
import os
from collections.abc import Mapping
from typing import Any, Dict, Iterator, Tuple

import torch

from ..parts.base import TensorSpec
from .safetensors_io import save_file

DEFAULT_SEED = 42          # as RBITNET_TOY_SEED's default, inference.rs:35


def _tensor_seed(seed: int, name: str) -> int:
    digest = hashlib.sha256(f"{int(seed)}:{name}".encode()).digest()
    return int.from_bytes(digest[:8], "little") & ((1 << 63) - 1)


def random_tensor(name: str, spec: TensorSpec, seed: int, std: float, norm_std: float,
                  dtype: torch.dtype, device: Any = "cpu") -> torch.Tensor:
    """One tensor's values.  Generated in float32 and rounded once to `dtype`
    (gains stay float32 only if `dtype` is float32: a stored model has one
    floating type).  CPU and GPU generators give different streams; a folder
    written on one device is the same for every reader."""
    g = torch.Generator(device=device)
    g.manual_seed(_tensor_seed(seed, name))
    if spec.role == "table":
        raise ValueError(f"no random rule for integer table {name!r}")
    t = torch.randn(spec.shape, generator=g, device=device, dtype=torch.float32)
    if spec.init == "ones_normal":
        t = 1.0 + norm_std * t
    else:
        t = std * t
    return t.to(dtype)


def random_tensors(expected: Dict[str, TensorSpec], seed: int, std: float = 0.02, norm_std: float = 0.02,
                   dtype: torch.dtype = torch.bfloat16, device: Any = "cpu") -> Iterator[Tuple[str, torch.Tensor]]:
    for name, spec in expected.items():
        yield name, random_tensor(name, spec, seed, std, norm_std, dtype, device)


class RandomTensors(Mapping):
    """name -> tensor, each drawn when it is asked for and not kept: a model far
    larger than its biggest tensor can be filled without holding a second copy."""

    def __init__(self, expected: Dict[str, TensorSpec], seed: int, std: float = 0.02, norm_std: float = 0.02,
                 dtype: torch.dtype = torch.bfloat16, device: Any = "cpu"):
        self._expected, self._args = expected, (seed, std, norm_std, dtype, device)

    def __getitem__(self, name: str) -> torch.Tensor:
        return random_tensor(name, self._expected[name], *self._args)

    def __iter__(self):
        return iter(self._expected)

    def __len__(self) -> int:
        return len(self._expected)


def write_random_model(folder: str, config: Any, seed: int = DEFAULT_SEED, std: float = 0.02,
                       norm_std: float = 0.02, dtype: torch.dtype = torch.bfloat16) -> str:
    """config (dict, or path of a config.json) + seed -> folder with config.json
    and model.safetensors.  Returns the folder."""
    from ..config import load_config
    from ..engine.model import expected_tensors

    if not isinstance(config, dict):
        path = os.path.join(config, "config.json") if os.path.isdir(config) else config
        with open(path) as f:
            config = json.load(f)
    cfg, spec = load_config(config)
    expected = expected_tensors(spec)
    os.makedirs(folder, exist_ok=True)
    raw = dict(config)                    # the caller's keys are kept as they are
    raw.setdefault("architectures", [spec.architecture])
    raw["torch_dtype"] = {torch.bfloat16: "bfloat16", torch.float32: "float32"}[dtype]
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(raw, f, indent=2)
    layout = {n: (dtype, tuple(s.shape)) for n, s in expected.items()}
    save_file(os.path.join(folder, "model.safetensors"),
              random_tensors(expected, seed, std, norm_std, dtype),
              metadata={"format": "pt", "seed": str(seed), "init_std": str(std), "norm_std": str(norm_std)},
              layout=layout)
    return folder
