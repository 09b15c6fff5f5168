"""One registry from an architecture's name to its configuration class.

config.json's `architectures[0]` chooses the class; the class turns the file's
keys into a `ModelSpec`.  The reference has no such table: it reads `llama.*`
keys whatever `general.architecture` says (gguf/bitnet_meta.rs:27-28) and uses
the name only as a label (gguf/parse.rs:222-234).

A configuration class has: `from_dict(dict)`, `to_dict()`, `to_spec()` and
optionally `tensor_aliases(name) -> [alternate names]` and `with_tensor_names(names)
-> configuration` (what the names in a weight file decide where config.json is silent).
"""
from __future__ import annotations

import json
import os
from typing import Any, Dict, Iterable, Optional, Tuple

from ..errors import ConfigError
from .llama import LlamaConfig
from .spec import ModelSpec

_ARCHITECTURES: Dict[str, Any] = {}


def register_architecture(name: str, config_class: Any) -> None:
    _ARCHITECTURES[name] = config_class


def registered_architectures():
    return sorted(_ARCHITECTURES)


def config_class_for(name: str) -> Any:
    if name not in _ARCHITECTURES:
        raise ConfigError(
            f"unknown architecture {name!r}; registered: {', '.join(registered_architectures())}")
    return _ARCHITECTURES[name]


def architecture_of(config: Dict[str, Any]) -> str:
    archs = config.get("architectures")
    if isinstance(archs, list) and archs:
        return str(archs[0])
    if isinstance(archs, str):
        return archs
    # a GGUF-style dump names it general.architecture = "llama" (gguf/parse.rs:222)
    model_type = config.get("model_type", config.get("general.architecture"))
    if model_type == "llama":
        return "LlamaForCausalLM"
    raise ConfigError("config.json names no architecture (key 'architectures')")


def load_config(path_or_dict: Any, tensor_names: Optional[Iterable[str]] = None) -> Tuple[Any, ModelSpec]:
    """config.json (a folder, a file or an already parsed dict) -> (typed
    configuration, spec).  tensor_names: the names in the weight file that goes with it."""
    if isinstance(path_or_dict, dict):
        raw = path_or_dict
    else:
        path = path_or_dict
        if os.path.isdir(path):
            path = os.path.join(path, "config.json")
        if not os.path.isfile(path):
            raise ConfigError(f"no config.json at {path}")
        with open(path) as f:
            try:
                raw = json.load(f)
            except json.JSONDecodeError as e:
                raise ConfigError(f"{path} is not valid JSON: {e}") from None
        if not isinstance(raw, dict):
            raise ConfigError(f"{path} does not hold a JSON object")
    cls = config_class_for(architecture_of(raw))
    cfg = cls.from_dict(raw)
    if tensor_names is not None and hasattr(cfg, "with_tensor_names"):
        cfg = cfg.with_tensor_names(list(tensor_names))
    return cfg, cfg.to_spec()


register_architecture("LlamaForCausalLM", LlamaConfig)
