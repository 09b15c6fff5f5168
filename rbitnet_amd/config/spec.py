"""Architecture-blind description of a model: which parts, in which order.

A configuration class (one per architecture, see `llama.py`) turns its own
config.json keys into a `ModelSpec`.  Everything below the configuration layer
(the loader, the parts, the cache, the step function) reads only the spec, so no
part knows which model it is in.

A `PartSpec` is a kind name plus parameters; the kind is looked up in the part
registries of `rbitnet_amd.parts`.  A `LayerSpec` holds the parts of one block
and the prefix under which its tensors are stored.  `ModelSpec.schedule` is the
order in which layers run: a list of indices into `layers`, which may name a
layer twice.  A mixer whose parameters hold `cache_from = j` keeps no cache of
its own and reads the one layer `j` wrote.

The two ends of a model are parts too: `embedding` (token ids -> stream) and `head`
(stream -> logits).  A spec that does not name them gets the plain ones, built from
`embedding_name`, `final_norm`, `final_norm_name` and `head_name`: a table whose rows are
gathered, and a norm followed by a matrix (the table again when `head_name` is None).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional


@dataclass
class PartSpec:
    kind: str
    params: Dict[str, Any] = field(default_factory=dict)

    def __getitem__(self, key: str) -> Any:
        return self.params[key]

    def get(self, key: str, default: Any = None) -> Any:
        return self.params.get(key, default)


@dataclass
class LayerSpec:
    """One block.  `block` names the arrangement of the parts ("prenorm":
    x += mixer(norm1(x)); x += ffn(norm2(x)))."""
    prefix: str
    block: str
    mixer: PartSpec
    feed_forward: PartSpec
    norm1: PartSpec
    norm2: PartSpec
    # tensor-name segment of each part below `prefix`, e.g. {"mixer": "self_attn"}
    segments: Optional[Dict[str, str]] = None


@dataclass
class ModelSpec:
    architecture: str
    hidden_size: int
    vocab_size: int
    max_positions: int
    layers: List[LayerSpec]
    # the plain ends, by their tensors (see the module's text); a spec that names `embedding` and `head`
    # itself needs none of the four
    embedding_name: Optional[str] = None
    final_norm: Optional[PartSpec] = None
    final_norm_name: Optional[str] = None
    head_name: Optional[str] = None          # None: the head is the embedding table (tied)
    schedule: List[int] = field(default_factory=list)
    stop_token_ids: List[int] = field(default_factory=list)
    bos_token_id: Optional[int] = None
    # tensors that a weight file may hold without the model reading them
    optional_tensors: List[str] = field(default_factory=list)
    embedding: Optional[PartSpec] = None
    head: Optional[PartSpec] = None

    def __post_init__(self) -> None:
        if self.embedding is None:
            if self.embedding_name is None:
                raise ValueError("a model needs an embedding: name the part, or the table's tensor")
            self.embedding = PartSpec("table", {"name": self.embedding_name, "vocab_size": self.vocab_size})
        if self.head is None:
            if self.final_norm is None or self.final_norm_name is None:
                raise ValueError("a model needs a head: name the part, or the final norm and its tensor")
            self.head = PartSpec("linear", {"norm": self.final_norm, "norm_name": self.final_norm_name,
                                            "name": self.head_name, "vocab_size": self.vocab_size})
        if not self.schedule:
            self.schedule = list(range(len(self.layers)))
        for i in self.schedule:
            if not 0 <= i < len(self.layers):
                raise ValueError(f"schedule names layer {i}, but the model has {len(self.layers)} layers")
