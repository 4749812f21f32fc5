"""Matrix products of the parts: out (=|+=) a @ weight.T with weights [out_features, in_features]
as checkpoints store them (no bias).  The kernel is chosen by the operands' storage: 32-bit
operands take the exact kernel; bfloat16 operands take the matrix-core kernels where their
shape rules allow and the exact kernel otherwise.  `a` may be a norm not yet applied
(`NormedRows`); it is applied here, by the norm's own kernel (which also gathers the rows it names).
Applying it inside the product's kernel was measured and did not pay: as a prologue it costs what the
separate kernel costs, and commuted into the epilogue it makes the product's loop twice as slow."""
from __future__ import annotations

import torch

from ..kernels import ops
from .norm import NormedRows


def linear(a, weight: torch.Tensor, out: torch.Tensor, accumulate: bool = False, gated: bool = False) -> torch.Tensor:
    """gated: weight is [gate; up] interleaved by `ops.interleave_gate_up` and out = silu(gate) * up (bfloat16 only)."""
    if isinstance(a, NormedRows):
        a = a.materialize()
    if a.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and ops.gemm_bf16_supports(a, weight, out):
        return ops.gemm_bf16(a, weight, out, accumulate, gated, checked=True)
    if gated:
        raise ops.KernelError("the gated product exists for bfloat16 operands only")
    return ops.gemm_exact(a, weight, out, accumulate)


def activation_dtype_for(weight: torch.Tensor, compute_dtype: torch.dtype) -> torch.dtype:
    """What the input of a product with `weight` is stored as: bfloat16 only if both the compute
    dtype and the weight are; a weight kept in 32-bit gets 32-bit activations."""
    return torch.bfloat16 if compute_dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 else torch.float32
