"""Matrix products y = x W^T with W stored [out, in] row-major, as the reference's
matvec loops read it (crates/bitnet-core/src/llama/model.rs:67-91).  No biases.

float32 operands run on the vector units in true 32-bit arithmetic; bfloat16
operands run on the matrix cores with float32 accumulation when the inner size
is a multiple of 8 (16-byte rows), else through the same generic kernel.

A product's result may be meant for the residual stream (`linear_to_stream`), and the tokens
may come as `GainedRows`, which such a product left for the norm after it.  With few tokens
on the matrix cores the products do the sums and the norms themselves and no kernel runs
between them; otherwise the caller is left with the sum and the rows are normalised first.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..errors import KernelError
from .norm import GainedRows

GATE_BLOCK = 16     # rows per block when gate and up rows are interleaved for the fused epilogue


def uses_matrix_cores(dtype: torch.dtype, k: int) -> bool:
    return dtype == torch.bfloat16 and k % 8 == 0


# False (tests and measurements set it): sums and norms stay kernels of their own
FOLD_INTO_PRODUCTS = True


def _few(lib, x, w: torch.Tensor) -> bool:
    """Whether the kernel for a few tokens, which folds its neighbours in, takes this product."""
    m, k = x.shape
    return FOLD_INTO_PRODUCTS and uses_matrix_cores(x.dtype, k) and lib.gemm_bf16_few_ok(m, w.shape[0], k)


def _from_gained(lib, x: GainedRows, w: torch.Tensor, out: torch.Tensor, epilogue: int) -> None:
    lib.gemm_bf16_few(x.gained, w, out, epilogue, squares=x.squares, eps=x.eps, rows=x.rows)


def linear(lib, x, w: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """[M, K] x [N, K]^T -> [M, N] in `out_dtype`."""
    m, k = x.shape
    n = w.shape[0]
    out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    if m == 0:
        return out
    if isinstance(x, GainedRows):
        if _few(lib, x, w):
            _from_gained(lib, x, w, out, 0)
            return out
        x = x.tensor()
    if uses_matrix_cores(x.dtype, k):
        lib.gemm_bf16(x, w, out, 0)
    else:
        if x.dtype == torch.float32 and out_dtype != torch.float32:
            raise KernelError("a float32 product has a float32 result")
        lib.gemm_generic(x, w, out)
    return out


def linear_or_terms(lib, x, w: torch.Tensor) -> torch.Tensor:
    """x W^T in float32 for a reader that adds up terms itself: [M, N], or [P, M, N] where the
    product's kernel cut K into P slices (their sums are then not added by a kernel of their own)."""
    if (not isinstance(x, GainedRows) and x.shape[0] > 0 and uses_matrix_cores(x.dtype, x.shape[1])
            and lib.gemm_bf16_terms_count(x.shape[0], w.shape[0], x.shape[1]) > 1):
        return lib.gemm_bf16_terms(x, w)
    return linear(lib, x, w, torch.float32)


def linear_to_stream(lib, x: torch.Tensor, w: torch.Tensor, stream: Optional[torch.Tensor], next_norm=None):
    """x W^T as a float32 term of the residual stream [M, N].  Without a stream, or where the
    product cannot add to it itself, the term comes back; as the [P, M, N] partial sums of the
    kernel's K slices where there are such and the norm that follows `adds_terms`.  Otherwise
    the product is added, and what comes back is None, or, if the norm that follows folds into
    products, the `GainedRows` for it."""
    if stream is None or x.shape[0] == 0 or not _few(lib, x, w):
        m, k = x.shape
        if (next_norm is not None and getattr(next_norm, "adds_terms", False) and uses_matrix_cores(x.dtype, k)
                and lib.gemm_bf16_terms_count(m, w.shape[0], k) > 1):
            return lib.gemm_bf16_terms(x, w)        # [P, M, N]: the norm adds them up with the stream
        return linear(lib, x, w, torch.float32)
    if next_norm is None or not getattr(next_norm, "folds_into_products", False):
        lib.gemm_bf16_few(x, w, stream, 2)
        return None
    m, n = stream.shape
    gained = torch.empty((m, n), dtype=torch.bfloat16, device=stream.device)
    squares = torch.empty((m, (n + 15) // 16), dtype=torch.float32, device=stream.device)
    lib.gemm_bf16_few(x, w, stream, 3, gain=next_norm.weight, gained=gained, squares_out=squares)
    return GainedRows(next_norm, stream, gained, squares)


def can_fuse_gate(dtype: torch.dtype, k: int, ff: int) -> bool:
    """Whether silu(gate) * up can be computed in the product's epilogue."""
    return uses_matrix_cores(dtype, k) and ff % GATE_BLOCK == 0


def pack_gate_up(lib, gate: torch.Tensor, up: torch.Tensor, fused: bool) -> torch.Tensor:
    """One matrix for both products.  Plain: gate rows, then up rows.  Fused: blocks of
    16 gate rows followed by the 16 up rows of the same columns, so that one lane of the
    matrix-core tile holds a gate value and its up value."""
    ff, k = gate.shape
    out = torch.empty((2 * ff, k), dtype=gate.dtype, device=gate.device)
    if fused:
        lib.place_rows(gate.contiguous(), out, row0=0, block=GATE_BLOCK, period=2 * GATE_BLOCK)
        lib.place_rows(up.contiguous(), out, row0=GATE_BLOCK, block=GATE_BLOCK, period=2 * GATE_BLOCK)
    else:
        lib.place_rows(gate.contiguous(), out, row0=0)
        lib.place_rows(up.contiguous(), out, row0=ff)
    return out


def gated_linear(lib, x, w_packed: torch.Tensor, ff: int, fused: bool) -> torch.Tensor:
    """silu(x Wg^T) * (x Wu^T) -> [M, ff] in x's dtype."""
    m = x.shape[0]
    out = torch.empty((m, ff), dtype=x.dtype, device=x.device)
    if m == 0:
        return out
    if isinstance(x, GainedRows):
        if fused and _few(lib, x, w_packed):
            _from_gained(lib, x, w_packed, out, 1)
            return out
        x = x.tensor()
    if fused:
        lib.gemm_bf16(x, w_packed, out, 1)
    else:
        gu = linear(lib, x, w_packed, torch.float32)
        lib.swiglu(gu, out)
    return out
