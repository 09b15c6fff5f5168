"""Weights by tensor name, checked against what the model's parts declare.

The reference loads each tensor by a list of alternate names
(`tensor_first_of`, crates/bitnet-core/src/gguf/parse.rs:60-62, used at
llama/model.rs:146-179) and fails at the first missing one or wrong element
count (model.rs:55-57, 181-194).  Here every tensor is looked up first and ONE
error lists everything that is wrong: missing tensors (with the names tried),
unexpected tensors, and wrong shapes (full shapes, not element counts).

Tensors come back in the element type they are stored in: bfloat16 stays
bfloat16, 32-bit stays 32-bit, float16 is widened to float32 (exact), 64-bit
integers become int32 (after a range check).  The model casts by role.
"""
from __future__ import annotations

from typing import Callable, Dict, Iterable, List, Optional, Tuple

import torch

from ..errors import WeightError
from ..parts.base import TensorSpec
from .safetensors_io import WeightFolder

_MAX_LISTED = 12


def _listing(items: List[str]) -> str:
    shown = items[:_MAX_LISTED]
    more = len(items) - len(shown)
    return "\n    " + "\n    ".join(shown) + (f"\n    ... and {more} more" if more > 0 else "")


def resolve_names(expected: Dict[str, TensorSpec], available: Iterable[str],
                  aliases: Optional[Callable[[str], List[str]]] = None,
                  optional: Iterable[str] = ()) -> Tuple[Dict[str, str], List[str], List[str]]:
    """expected name -> stored name; plus (missing, unexpected)."""
    have = set(available)
    used = set()
    mapping: Dict[str, str] = {}
    missing: List[str] = []
    for name in expected:
        tried = [name] + (aliases(name) if aliases else [])
        hit = next((t for t in tried if t in have), None)
        if hit is None:
            missing.append(f"{name} (tried {tried})" if len(tried) > 1 else name)
        else:
            mapping[name] = hit
            used.add(hit)
    optional_hits = set()
    for name in optional:
        for t in [name] + (aliases(name) if aliases else []):
            if t in have:
                optional_hits.add(t)
    unexpected = sorted(have - used - optional_hits)
    return mapping, missing, unexpected


def load_weights(folder: str, expected: Dict[str, TensorSpec],
                 aliases: Optional[Callable[[str], List[str]]] = None,
                 ignored: Iterable[str] = (), strict: bool = True) -> Dict[str, torch.Tensor]:
    """All expected tensors, by expected name, as CPU tensors in stored type.

    `ignored` names tensors that may be present without being used (an output
    matrix beside tied embeddings).  Anything else that is present and not
    expected is an error when `strict`."""
    store = WeightFolder(folder)
    mapping, missing, unexpected = resolve_names(expected, store.names(), aliases, ignored)
    wrong: List[str] = []
    for name, stored in mapping.items():
        dtype, shape = store.info(stored)
        want = tuple(expected[name].shape)
        if tuple(shape) != want:
            wrong.append(f"{name}: expected {list(want)}, found {list(shape)}")
        elif expected[name].role == "table" and dtype not in ("I32", "I64"):
            wrong.append(f"{name}: expected integers, found {dtype}")
        elif expected[name].role != "table" and dtype in ("I32", "I64"):
            wrong.append(f"{name}: expected floating point, found {dtype}")
    problems = []
    if missing:
        problems.append(f"  missing tensors ({len(missing)}):" + _listing(missing))
    if unexpected and strict:
        problems.append(f"  unexpected tensors ({len(unexpected)}):" + _listing(unexpected))
    if wrong:
        problems.append(f"  wrong shapes ({len(wrong)}):" + _listing(wrong))
    if problems:
        raise WeightError(f"weights in {folder} do not match the model:\n" + "\n".join(problems))
    out: Dict[str, torch.Tensor] = {}
    for name, stored in mapping.items():
        t = store.tensor(stored)
        if t.dtype == torch.float16:
            t = t.to(torch.float32)
        elif t.dtype == torch.int64:
            if t.numel() and (int(t.max()) > 2**31 - 1 or int(t.min()) < -2**31):
                raise WeightError(f"{name}: integer table does not fit 32 bits")
            t = t.to(torch.int32)
        out[name] = t
    return out
