"""Matrix products of the parts: out (=|+=) a @ weight.T with weights [out_features, in_features]
as checkpoints store them (no bias).  The kernel is chosen by the operands' storage: 32-bit
operands take the exact kernel; bfloat16 operands take the matrix-core kernels where their
shape rules allow and the exact kernel otherwise.  `a` may be a norm not yet applied
(`NormedRows`); it is applied here, by the norm's own kernel (which also gathers the rows it names).
Applying it inside the product's kernel was measured and did not pay: as a prologue it costs what the
separate kernel costs, and commuted into the epilogue with the product reading the 32-bit rows it
makes the product's loop twice as slow.  What pays, for a few rows, is to split it over the two
products around it (`HandedRows`, `linear_onto`): the one that writes the rows also writes them
times the norm's weights in bfloat16 and the pieces of their sums of squares, the one that reads them
multiplies its results by the rows' rsqrt(mean square + eps)."""
from __future__ import annotations

import torch

from ..kernels import ops
from .norm import HandedRows, NormedRows


def linear(a, weight: torch.Tensor, out: torch.Tensor, accumulate: bool = False, gated: bool = False) -> torch.Tensor:
    """gated: weight is [gate; up] interleaved by `ops.interleave_gate_up` and out = silu(gate) * up (bfloat16 only)."""
    if isinstance(a, HandedRows):
        if (weight.dtype == torch.bfloat16 and ops.gemm_bf16_supports(a.scaled, weight, out)
                and ops.gemm_bf16_takes_norm(a.scaled.shape[0], weight.shape[0], weight.shape[1], gated)):
            return ops.gemm_bf16(a.scaled, weight, out, accumulate, gated, checked=True, norm_in=(a.squares, a.eps))
    if isinstance(a, NormedRows):
        a = a.materialize()
    if a.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and ops.gemm_bf16_supports(a, weight, out):
        return ops.gemm_bf16(a, weight, out, accumulate, gated, checked=True)
    if gated:
        raise ops.KernelError("the gated product exists for bfloat16 operands only")
    return ops.gemm_exact(a, weight, out, accumulate)


def linear_onto(a: torch.Tensor, weight: torch.Tensor, residual: torch.Tensor, then=None):
    """residual += a @ weight.T.  `then`: the norm that reads `residual` next, if it and its reader can take it half applied
    (see `HandedRows`); the product then also does the norm's share and the `HandedRows` are returned, None otherwise."""
    if (then is not None and a.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and residual.dtype == torch.float32
            and residual.is_contiguous() and ops.gemm_bf16_supports(a, weight, residual)):
        rows, width = residual.shape
        parts = ops.gemm_bf16_norm_parts(rows, weight.shape[0], weight.shape[1])
        if parts:
            scaled = torch.empty((rows, width), dtype=torch.bfloat16, device=residual.device)
            squares = torch.empty((rows, parts), dtype=torch.float32, device=residual.device)
            ops.gemm_bf16(a, weight, residual, accumulate=True, checked=True, norm_out=(then.handed_weight(), scaled, squares))
            return HandedRows(then, residual, scaled, squares)
    linear(a, weight, residual, accumulate=True)
    return None


def activation_dtype_for(weight: torch.Tensor, compute_dtype: torch.dtype) -> torch.dtype:
    """What the input of a product with `weight` is stored as: bfloat16 only if both the compute
    dtype and the weight are; a weight kept in 32-bit gets 32-bit activations."""
    return torch.bfloat16 if compute_dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 else torch.float32
