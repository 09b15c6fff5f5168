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
from .stream import GainedRows, norm_adds_terms, norm_folds

GATE_BLOCK = 16     # rows per block when gate and up rows are interleaved for the fused epilogue


class Matrix:
    """A weight matrix [N, K] as the product kernels read it.  `data` holds its N x K values, as N
    rows, or, `frag`, fragment-major: blocks of 1 KB (16 rows x 32 bfloat16 or 16 float32 columns) in
    the order [N / 16][K / columns], laid out as the matrix cores' row operand, so that a wave reads
    1 KB in a row per load and a decode step streams W past the caches (bfloat16: 6.0-6.8 TB/s against
    5.3-5.8 for rows).  bfloat16 matrices with N % 16 == 0 and K % 64 == 0 and float32 ones with
    N % 16 == 0 and K % 128 == 0 are stored so; `pack_rows` decides."""

    def __init__(self, data: torch.Tensor, frag: bool = False):
        self.data, self.frag = data, bool(frag)
        self.shape, self.dtype, self.device = data.shape, data.dtype, data.device


def _data(w):
    return (w.data, w.frag) if isinstance(w, Matrix) else (w, False)


def fragment_major_ok(dtype: torch.dtype, n: int, k: int) -> bool:
    """bfloat16: the matrix-core products read either layout when N % 16 == 0 and K % 64 == 0.  float32:
    with N % 16 == 0 and K % 128 == 0 every step's product runs on a kernel that reads it."""
    if dtype == torch.float32:
        return n % 16 == 0 and k % 128 == 0
    return dtype == torch.bfloat16 and n % 16 == 0 and k % 64 == 0


def pack_rows(lib, pieces, n: int, k: int, dtype: torch.dtype, device, frag_allowed: bool = True) -> Matrix:
    """One matrix [n, k] from `pieces`: (tensor [rows, k], first row, block, period) as
    `place_rows` takes them.  Stored fragment-major where the matrix-core kernels can read that."""
    frag = frag_allowed and fragment_major_ok(dtype, n, k)
    out = torch.empty((n, k), dtype=dtype, device=device)
    for t, row0, block, period in pieces:
        lib.place_rows(t.contiguous(), out, row0=row0, block=block, period=period, frag=frag)
    return Matrix(out, frag)


def uses_matrix_cores(dtype: torch.dtype, k: int) -> bool:
    return dtype == torch.bfloat16 and k % 8 == 0


# False (tests and measurements set it): sums and norms stay kernels of their own
FOLD_INTO_PRODUCTS = True


def _few(lib, x, w) -> bool:
    """Whether the kernel for a few tokens, which folds its neighbours in, takes this product."""
    m, k = x.shape
    return FOLD_INTO_PRODUCTS and uses_matrix_cores(x.dtype, k) and lib.gemm_bf16_few_ok(m, w.shape[0], k)


def _from_gained(lib, x: GainedRows, w, out: torch.Tensor, epilogue: int) -> None:
    wd, frag = _data(w)
    lib.gemm_bf16_few(x.gained, wd, out, epilogue, squares=x.squares, eps=x.eps, rows=x.rows, w_frag=frag)


def linear(lib, x, w, out_dtype: torch.dtype) -> torch.Tensor:
    """[M, K] x [N, K]^T -> [M, N] in `out_dtype`.  w: a tensor of N rows, or a `Matrix`."""
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
    wd, frag = _data(w)
    if uses_matrix_cores(x.dtype, k):
        lib.gemm_bf16(x, wd, out, 0, w_frag=frag)
    else:
        if frag and x.dtype != torch.float32:
            raise KernelError("a fragment-major bfloat16 matrix is for the matrix-core products only")
        if x.dtype == torch.float32 and out_dtype != torch.float32:
            raise KernelError("a float32 product has a float32 result")
        lib.gemm_generic(x, wd, out, w_frag=frag)
    return out


def linear_or_terms(lib, x, w) -> torch.Tensor:
    """x W^T in float32 for a reader that adds up terms itself: [M, N], or [P, M, N] where the
    product's kernel cut K into P slices (their sums are then not added by a kernel of their own)."""
    if (not isinstance(x, GainedRows) and x.shape[0] > 0 and uses_matrix_cores(x.dtype, x.shape[1])
            and lib.gemm_bf16_terms_count(x.shape[0], w.shape[0], x.shape[1]) > 1):
        wd, frag = _data(w)
        return lib.gemm_bf16_terms(x, wd, w_frag=frag)
    return linear(lib, x, w, torch.float32)


def linear_to_stream(lib, x: torch.Tensor, w, stream: Optional[torch.Tensor], next_norm=None):
    """x W^T as a float32 term of the residual stream [M, N].  Without a stream, or where the
    product cannot add to it itself, the term comes back; as the [P, M, N] partial sums of the
    kernel's K slices where there are such and the norm that follows `adds_terms`.  Otherwise
    the product is added, and what comes back is None, or, if the norm that follows folds into
    products, the `GainedRows` for it."""
    wd, frag = _data(w)
    if stream is None or x.shape[0] == 0 or not _few(lib, x, w):
        m, k = x.shape
        if (norm_adds_terms(next_norm) and uses_matrix_cores(x.dtype, k)
                and lib.gemm_bf16_terms_count(m, w.shape[0], k) > 1):
            return lib.gemm_bf16_terms(x, wd, w_frag=frag)        # [P, M, N]: the norm adds them up with the stream
        return linear(lib, x, w, torch.float32)
    if not norm_folds(next_norm):
        lib.gemm_bf16_few(x, wd, stream, 2, w_frag=frag)
        return None
    m, n = stream.shape
    gained = torch.empty((m, n), dtype=torch.bfloat16, device=stream.device)
    squares = torch.empty((m, (n + 15) // 16), dtype=torch.float32, device=stream.device)
    lib.gemm_bf16_few(x, wd, stream, 3, gain=next_norm.weight, gained=gained, squares_out=squares, w_frag=frag)
    return GainedRows(next_norm, stream, gained, squares)


def can_fuse_gate(dtype: torch.dtype, k: int, ff: int) -> bool:
    """Whether silu(gate) * up can be computed in the product's epilogue."""
    return uses_matrix_cores(dtype, k) and ff % GATE_BLOCK == 0


def pack_gate_up(lib, gate: torch.Tensor, up: torch.Tensor, fused: bool, frag_allowed: bool = True) -> Matrix:
    """One matrix for both products.  Plain: gate rows, then up rows.  Fused: blocks of
    16 gate rows followed by the 16 up rows of the same columns, so that one lane of the
    matrix-core tile holds a gate value and its up value."""
    ff, k = gate.shape
    if fused:
        pieces = [(gate, 0, GATE_BLOCK, 2 * GATE_BLOCK), (up, GATE_BLOCK, GATE_BLOCK, 2 * GATE_BLOCK)]
    else:
        pieces = [(gate, 0, None, None), (up, ff, None, None)]
    return pack_rows(lib, pieces, 2 * ff, k, gate.dtype, gate.device, frag_allowed)


def gated_linear(lib, x, w_packed, ff: int, fused: bool) -> torch.Tensor:
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
        wd, frag = _data(w_packed)
        lib.gemm_bf16(x, wd, out, 1, w_frag=frag)
    else:
        gu = linear(lib, x, w_packed, torch.float32)
        lib.swiglu(gu, out)
    return out
