"""The residual stream and who adds to it: the one place that knows.

The stream x is float32 [T, E].  A sublayer is `x += part(norm(x))`
(crates/bitnet-core/src/llama/model.rs:236-307); the sum is not done where the reference
does it but by whoever can do it without a pass of its own over memory: the norm that follows
(its kernel adds `pending` to x before it normalises), or, in a step of few tokens, the
part's last product (which adds its float32 sums to x in its epilogue and leaves the rows
prepared for the norm that follows, `GainedRows`).  What a sublayer has not yet added is
`pending`, and it takes one of four forms:

    None            nothing: the stream holds the sum already
    tensor [T, E]   a float32 term still to be added
    tensor [P,T,E]  P terms, the K slices of a product, to be added up in their order
    GainedRows      nothing to add, and the rows as the next norm's kernel would read them

What a part or a norm can do, it says with class attributes; a part without any gets and
returns plain tensors, a norm without any does every sum and every normalisation in its own
`forward`:

    part.adds_to_stream       forward takes stream=x and next_norm, and may return any form above
    part.takes_gained_rows    forward's input may be GainedRows instead of a tensor
    norm.adds_terms           forward's delta may be [P, T, E]
    norm.folds_into_products  the norm is x * weight / sqrt(mean x^2 + eps) with `weight`, `eps`
                              and `size`, so that products may do its work (GainedRows)
    block.takes_next_norm     forward takes next_norm: the first norm of whatever runs after it
    block.first_norm          that norm, for the block before

A block arrangement calls `sublayer` once per part and returns the last `pending`; `run_blocks`
runs blocks in schedule order; a product that ends a part (`linear.linear_to_stream`) asks
`norm_adds_terms` and `norm_folds` what it may leave.  Nothing else reads the attributes above.
"""
from __future__ import annotations

from typing import Optional, Sequence

import torch


class GainedRows:
    """Rows of the float32 stream `x` (all, or those `rows` names) as a product left them for
    `norm`: gained [T, E] = bf16(x * gain) and squares [T, ceil(E / 16)], the sums of x^2 over
    every 16 columns.  What is left of the norm is one factor per row.  `linear` takes them as
    tokens; tensor() normalises the rows with the norm's own kernel instead.  shape, dtype and
    device are those of the normalised rows."""

    def __init__(self, norm, x: torch.Tensor, gained: torch.Tensor, squares: torch.Tensor,
                 rows: Optional[torch.Tensor] = None):
        self.norm = norm
        self.x = x
        self.gained = gained
        self.squares = squares
        self.rows = rows
        self.eps = norm.eps
        self.shape = (x.shape[0] if rows is None else rows.shape[0], norm.size)
        self.dtype = norm.env.dtype
        self.device = x.device

    def select(self, rows: Optional[torch.Tensor]) -> "GainedRows":
        if rows is None:
            return self
        if self.rows is not None:
            raise ValueError("rows were chosen already")
        return GainedRows(self.norm, self.x, self.gained, self.squares, rows)

    def tensor(self) -> torch.Tensor:
        return self.norm.forward(self.x, None, self.rows)


def normed_for(part, norm, x: torch.Tensor, pending, rows: Optional[torch.Tensor] = None):
    """The input of `part`: the stream x, with `pending` added if that is a tensor, normalised
    by `norm` (all rows, or `rows`).  GainedRows that were made for this norm go on as they are
    to a part that takes them."""
    if isinstance(pending, GainedRows):
        if pending.norm is norm and getattr(part, "takes_gained_rows", False):
            return pending.select(rows)
        return norm.forward(x, None, rows)         # the stream holds the sum already
    return norm.forward(x, pending, rows)


def sublayer(part, norm, x: torch.Tensor, pending, next_norm, *args):
    """x += part(norm(x + pending)), as far as it is done here: returns what is still pending.
    `args` are the part's own (ctx and view for a mixer, ctx for a feed-forward); `next_norm` is
    the norm that will read the stream next (None: unknown)."""
    h = normed_for(part, norm, x, pending)
    if getattr(part, "adds_to_stream", False):
        return part.forward(h, *args, stream=x, next_norm=next_norm)
    return part.forward(h, *args)


def run_blocks(blocks: Sequence, schedule: Sequence[int], x: torch.Tensor, ctx, cache, last_norm=None):
    """The blocks in schedule order on the stream x; returns what the last one left pending.
    last_norm: the norm that reads the stream after the last block."""
    pending = None
    for place, i in enumerate(schedule):
        block = blocks[i]
        view = cache.view(place, ctx.block_tables)
        if getattr(block, "takes_next_norm", False):
            after = blocks[schedule[place + 1]] if place + 1 < len(schedule) else None
            next_norm = last_norm if after is None else getattr(after, "first_norm", None)
            pending = block.forward(x, pending, ctx, view, next_norm=next_norm)
        else:
            pending = block.forward(x, pending, ctx, view)
    return pending


def norm_adds_terms(norm) -> bool:
    """Whether a product before `norm` may leave its K slices' sums [P, T, E] for it to add up."""
    return norm is not None and bool(getattr(norm, "adds_terms", False))


def norm_folds(norm) -> bool:
    """Whether a product before `norm` may add to the stream itself and leave `GainedRows`."""
    return norm is not None and bool(getattr(norm, "folds_into_products", False))
