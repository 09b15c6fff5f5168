"""Matrix products y = x W^T with W stored [out, in] row-major, as the reference's
matvec loops read it (crates/bitnet-core/src/llama/model.rs:67-91).  No biases.

float32 operands run on the vector units in true 32-bit arithmetic; bfloat16
operands run on the matrix cores with float32 accumulation when the inner size
is a multiple of 8 (16-byte rows), else through the same generic kernel.
"""
from __future__ import annotations

import torch

from ..errors import KernelError

GATE_BLOCK = 16     # rows per block when gate and up rows are interleaved for the fused epilogue


def uses_matrix_cores(dtype: torch.dtype, k: int) -> bool:
    return dtype == torch.bfloat16 and k % 8 == 0


def linear(lib, x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """[M, K] x [N, K]^T -> [M, N] in `out_dtype`."""
    m, k = x.shape
    n = w.shape[0]
    out = torch.empty((m, n), dtype=out_dtype, device=x.device)
    if m == 0:
        return out
    if uses_matrix_cores(x.dtype, k):
        lib.gemm_bf16(x, w, out, 0)
    else:
        if x.dtype == torch.float32 and out_dtype != torch.float32:
            raise KernelError("a float32 product has a float32 result")
        lib.gemm_generic(x, w, out)
    return out


def can_fuse_gate(dtype: torch.dtype, k: int, ff: int) -> bool:
    """Whether silu(gate) * up can be computed in the product's epilogue."""
    return uses_matrix_cores(dtype, k) and ff % GATE_BLOCK == 0


def pack_gate_up(gate: torch.Tensor, up: torch.Tensor, fused: bool) -> torch.Tensor:
    """One matrix for both products.  Plain: gate rows, then up rows.  Fused: blocks of
    16 gate rows followed by the 16 up rows of the same columns, so that one lane of the
    matrix-core tile holds a gate value and its up value."""
    ff, k = gate.shape
    if not fused:
        return torch.cat([gate, up], dim=0).contiguous()
    g = gate.reshape(ff // GATE_BLOCK, GATE_BLOCK, k)
    u = up.reshape(ff // GATE_BLOCK, GATE_BLOCK, k)
    return torch.stack([g, u], dim=1).reshape(2 * ff, k).contiguous()


def gated_linear(lib, x: torch.Tensor, w_packed: torch.Tensor, ff: int, fused: bool) -> torch.Tensor:
    """silu(x Wg^T) * (x Wu^T) -> [M, ff] in x's dtype."""
    m = x.shape[0]
    out = torch.empty((m, ff), dtype=x.dtype, device=x.device)
    if m == 0:
        return out
    if fused:
        lib.gemm_bf16(x, w_packed, out, 1)
    else:
        gu = linear(lib, x, w_packed, torch.float32)
        lib.swiglu(gu, out)
    return out
