"""Random weights from a configuration and a seed, as a model folder or in memory.

The reference's counterpart is its toy model, every value of which a seed fixes
(crates/bitnet-core/src/model/toy.rs:16-30, seed from RBITNET_TOY_SEED with
default 42, inference.rs:31-36).  Here every tensor the model's parts declare is
drawn by name: matrices N(0, std), norm gains 1 + N(0, norm_std).  Element i of a
tensor is a function of (seed, tensor name, i) alone, so the values depend neither
on the order of the tensors, nor on which others exist, nor on the device: the
GPU's fill kernel (csrc/weights_init.hip) and `normal_values` below, its twin on
the host, give the same bits, and a seed means one model whether it is drawn in
memory (`Engine.random`) or written to a folder and loaded.

    key  = the first 8 bytes (little endian) of sha256("<seed>:<name>")
    pair p = i // 2;  h = mix(key + (p + 1) * 0x9E3779B97F4A7C15)   (64-bit, wrapping)
    m = (h >> 32) + 1,  n = h & 0xffffffff
    radius = sqrt(-2 ln(m / 2^32)),  angle = 2 pi n / 2^32
    z = radius * cos(angle) for even i, radius * sin(angle) for odd i
    value = float32(mean + std * z), then rounded to bfloat16 where that is stored

Logarithm, sine and cosine are written out with float64 additions, multiplications,
divisions and a square root (each rounds the same way everywhere), in the same order
as in the kernel.
"""
from __future__ import annotations

import hashlib
import json
import os
from collections.abc import Mapping
from typing import Any, Dict, Iterator, Tuple

import numpy as np
import torch

from ..parts.base import TensorSpec
from .safetensors_io import save_file

DEFAULT_SEED = 42          # as RBITNET_TOY_SEED's default, inference.rs:35
_CHUNK = 1 << 21           # pairs drawn at a time on the host


def tensor_key(seed: int, name: str) -> int:
    digest = hashlib.sha256(f"{int(seed)}:{name}".encode()).digest()
    return int.from_bytes(digest[:8], "little")


def _mix64(z: np.ndarray) -> np.ndarray:
    z = z ^ (z >> np.uint64(30))
    z = z * np.uint64(0xBF58476D1CE4E5B9)
    z = z ^ (z >> np.uint64(27))
    z = z * np.uint64(0x94D049BB133111EB)
    return z ^ (z >> np.uint64(31))


def _log_unit(m_minus_1: np.ndarray) -> np.ndarray:
    """ln(m / 2^32) for integers m in [1, 2^32] (see log_unit in csrc/weights_init.hip)."""
    m = m_minus_1.astype(np.float64) + 1.0
    f, e = np.frexp(m)
    low = f < float("0.70710678118654752440")
    f = np.where(low, f * 2.0, f)
    e = np.where(low, e - 1, e)
    s = (f - 1.0) / (f + 1.0)
    s2 = s * s
    p = np.full_like(s, 1.0 / 23.0)
    for odd in (21.0, 19.0, 17.0, 15.0, 13.0, 11.0, 9.0, 7.0, 5.0, 3.0):
        p = p * s2 + 1.0 / odd
    p = p * s2 + 1.0
    return (e - 32).astype(np.float64) * float("0.69314718055994530942") + 2.0 * s * p


def _sincos_octant(x: np.ndarray):
    x2 = x * x
    p = np.full_like(x, 1.0 / 355687428096000.0)
    for sign, fact in ((-1, 1307674368000.0), (1, 6227020800.0), (-1, 39916800.0), (1, 362880.0), (-1, 5040.0),
                       (1, 120.0), (-1, 6.0)):
        p = p * x2 + 1.0 / fact if sign > 0 else p * x2 - 1.0 / fact
    p = p * x2 + 1.0
    s = x * p
    q = np.full_like(x, -1.0 / 6402373705728000.0)
    for sign, fact in ((1, 20922789888000.0), (-1, 87178291200.0), (1, 479001600.0), (-1, 3628800.0), (1, 40320.0),
                       (-1, 720.0), (1, 24.0), (-1, 2.0)):
        q = q * x2 + 1.0 / fact if sign > 0 else q * x2 - 1.0 / fact
    q = q * x2 + 1.0
    return s, q


def _normal_pairs(key: int, first_pair: int, n_pairs: int):
    with np.errstate(over="ignore"):
        p = np.arange(first_pair + 1, first_pair + n_pairs + 1, dtype=np.uint64)
        h = _mix64(np.uint64(key) + p * np.uint64(0x9E3779B97F4A7C15))
    hi = (h >> np.uint64(32)).astype(np.uint32)
    lo = (h & np.uint64(0xFFFFFFFF)).astype(np.uint32)
    radius = np.sqrt(-2.0 * _log_unit(hi))
    octant = lo >> np.uint32(29)
    r = (lo & np.uint32(0x1FFFFFFF)).astype(np.int64)
    t = np.where(octant & np.uint32(1), 0x20000000 - r, r)
    x = t.astype(np.float64) * (float("3.14159265358979323846") / 2147483648.0)
    s, c = _sincos_octant(x)
    swap = ((octant + np.uint32(1)) >> np.uint32(1)) & np.uint32(1)
    cosv = np.where(swap, s, c)
    sinv = np.where(swap, c, s)
    cosv = np.where(((octant + np.uint32(2)) >> np.uint32(2)) & np.uint32(1), -cosv, cosv)
    sinv = np.where(octant >> np.uint32(2), -sinv, sinv)
    return radius * cosv, radius * sinv


def normal_values(key: int, n: int, mean: float, std: float) -> np.ndarray:
    """float32 [n]: the host twin of the GPU's fill kernel."""
    out = np.empty(n, dtype=np.float32)
    n_pairs = (n + 1) // 2
    for first in range(0, n_pairs, _CHUNK):
        count = min(_CHUNK, n_pairs - first)
        z0, z1 = _normal_pairs(key, first, count)
        both = np.empty(2 * count, dtype=np.float64)
        both[0::2] = z0
        both[1::2] = z1
        both = (float(mean) + float(std) * both).astype(np.float32)
        lo = 2 * first
        hi = min(n, lo + 2 * count)
        out[lo:hi] = both[:hi - lo]
    return out


def random_tensor(name: str, spec: TensorSpec, seed: int, std: float, norm_std: float,
                  dtype: torch.dtype, device: Any = "cpu") -> torch.Tensor:
    """One tensor's values, generated in float32 and rounded once to `dtype`: on the GPU
    by the fill kernel, elsewhere by its host twin, with the same bits."""
    if spec.role == "table":
        raise ValueError(f"no random rule for integer table {name!r}")
    mean, scale = (1.0, norm_std) if spec.init == "ones_normal" else (0.0, std)
    key = tensor_key(seed, name)
    n = 1
    for d in spec.shape:
        n *= int(d)
    if torch.device(device).type == "cuda":
        from ..csrc.lib import kernels
        out = torch.empty(tuple(spec.shape), dtype=dtype, device=device)
        kernels().fill_normal(out, key, mean, scale)
        return out
    values = torch.from_numpy(normal_values(key, n, mean, scale)).reshape(tuple(spec.shape))
    return values.to(dtype)


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
                       norm_std: float = 0.02, dtype: torch.dtype = torch.bfloat16, device: Any = None) -> str:
    """config (dict, or path of a config.json) + seed -> folder with config.json
    and model.safetensors.  Returns the folder.  device: where the numbers are drawn (the
    same numbers everywhere; the GPU is far faster for large models); None: the GPU if there
    is one and the kernel library can be loaded, else the host."""
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
    if device is None:
        device = "cpu"
        if torch.cuda.is_available():
            try:                          # the GPU when its kernels can be had, else the host twin: the same numbers
                from ..csrc.lib import kernels
                kernels()
                device = "cuda:0"
            except Exception:
                pass
    save_file(os.path.join(folder, "model.safetensors"),
              ((n, t.cpu()) for n, t in random_tensors(expected, seed, std, norm_std, dtype, device)),
              metadata={"format": "pt", "seed": str(seed), "init_std": str(std), "norm_std": str(norm_std)},
              layout=layout)
    return folder
