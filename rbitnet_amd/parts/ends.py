"""The two ends of a model: what turns token ids into the residual stream, and what turns
the stream into logits.  Parts like the others: a kind in a registry, parameters, tensors of
their own, a forward; a model's forward is the embedding, the blocks in schedule order, the
head, and holds no stage of its own.  An architecture that scales its embeddings, or scales or
caps its logits, or computes them in another way, registers another kind.

Their tensors have no layer prefix: `tensor_specs` names them in full.

embedding "table" (crates/bitnet-core/src/llama/model.rs:229-232): x[t, :] = table[id[t], :].
    Parameters: name, vocab_size.
    Interface of an embedding: tensor_specs() / load(tensors) / forward(ctx) -> float32 [T, E]
    (ctx.token_ids int32 [T]); `table` if a head may share it.

head "linear" (model.rs:309-315): logits = W norm(x), on the asked rows only; W is the
    embedding's table when the parameters name no matrix (tied).
    Parameters: norm (a PartSpec), norm_name, name (None: tied), vocab_size.
    Interface of a head: tensor_specs() / load(tensors, embedding) /
    forward(x, pending, rows, ctx) -> float32 [len(rows), V], where x is the stream, `pending`
    what the last block left to be added (see stream.py) and rows the packed rows asked for;
    first_norm (optional): the norm it begins with, for the last block.
    step_bytes(element_size) (optional, both ends): the bytes of its tensors that a step reads
    in full (default: all of them).
"""
from __future__ import annotations

from typing import Dict, Optional

import torch

from ..errors import ConfigError
from .base import BuildEnv, Part, TensorSpec, build_part, register_embedding, register_head
from .linear import linear, pack_rows
from .stream import normed_for


class TableEmbedding(Part):
    graph_safe = True
    plan_safe = True

    def __init__(self, params: Dict, env: BuildEnv):
        self.env = env
        self.name = str(params["name"])
        self.vocab_size = int(params["vocab_size"])
        self.hidden = env.hidden_size
        self.table: Optional[torch.Tensor] = None

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        return {self.name: TensorSpec((self.vocab_size, self.hidden))}

    def load(self, tensors: Dict[str, torch.Tensor]) -> None:
        self.table = tensors[self.name]

    def step_bytes(self, element_size: int) -> int:
        return 0                      # the gather reads a few rows only

    def forward(self, ctx) -> torch.Tensor:
        x = torch.empty((ctx.n_tokens, self.hidden), dtype=torch.float32, device=self.table.device)
        self.env.lib.embed_gather(self.table, ctx.token_ids, x)
        return x


class LinearHead(Part):
    takes_gained_rows = True      # the output product takes what the last product left for the final norm

    def __init__(self, params: Dict, env: BuildEnv):
        self.env = env
        self.norm = build_part("norm", params["norm"], env)
        self.norm_name = str(params["norm_name"])
        self.name = params.get("name")
        self.vocab_size = int(params["vocab_size"])
        self.hidden = env.hidden_size
        self.weight = None

    @property
    def graph_safe(self) -> bool:
        return bool(getattr(self.norm, "graph_safe", False))

    @property
    def plan_safe(self) -> bool:
        return bool(getattr(self.norm, "plan_safe", False))

    @property
    def first_norm(self):
        return self.norm

    def _norm_names(self) -> Dict[str, str]:
        """full name -> the norm's own name of the tensor"""
        specs = self.norm.tensor_specs()
        if len(specs) == 1:
            return {self.norm_name: next(iter(specs))}
        base = self.norm_name.rsplit(".", 1)[0]
        return {f"{base}.{name}": name for name in specs}

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        own = self.norm.tensor_specs()
        out = {full: own[name] for full, name in self._norm_names().items()}
        if self.name is not None:
            out[str(self.name)] = TensorSpec((self.vocab_size, self.hidden))
        return out

    def load(self, tensors: Dict[str, torch.Tensor], embedding=None) -> None:
        self.norm.load({name: tensors[full] for full, name in self._norm_names().items()})
        if self.name is None:
            table = getattr(embedding, "table", None)
            if table is None or tuple(table.shape) != (self.vocab_size, self.hidden):
                raise ConfigError("a head without a matrix of its own needs an embedding whose table it can share")
            self.weight = table                 # tied: the table's rows are also read one by one, so it stays rows
            return
        w = tensors[str(self.name)]
        self.weight = pack_rows(self.env.lib, [(w, 0, None, None)], w.shape[0], w.shape[1], w.dtype, w.device,
                                not getattr(self.env, "generic_only", False))

    def step_bytes(self, element_size: int) -> int:
        gains = sum(4 * _numel(ts.shape) for ts in self.norm.tensor_specs().values())
        return gains + self.vocab_size * self.hidden * element_size        # tied or not, the matrix is read once

    def forward(self, x: torch.Tensor, pending, rows: torch.Tensor, ctx=None) -> torch.Tensor:
        xn = normed_for(self, self.norm, x, pending, rows)
        return linear(self.env.lib, xn, self.weight, torch.float32)


def _numel(shape) -> int:
    n = 1
    for s in shape:
        n *= int(s)
    return n


register_embedding("table", TableEmbedding)
register_head("linear", LinearHead)
