"""Matrix products of the parts: out (=|+=) a @ weight.T with weights [out_features, in_features]
as checkpoints store them (no bias).  The kernel is chosen by the operands' storage: 32-bit
operands take the exact kernel; bfloat16 operands take the matrix-core kernels where their
shape rules allow and the exact kernel otherwise."""
from __future__ import annotations

import torch

from ..kernels import ops


def linear(a: torch.Tensor, weight: torch.Tensor, out: torch.Tensor, accumulate: bool = False) -> torch.Tensor:
    if a.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and ops.gemm_bf16_supports(a, weight, out):
        return ops.gemm_bf16(a, weight, out, accumulate)
    return ops.gemm_exact(a, weight, out, accumulate)


def activation_dtype_for(weight: torch.Tensor, compute_dtype: torch.dtype) -> torch.dtype:
    """What the input of a product with `weight` is stored as: bfloat16 only if both the compute
    dtype and the weight are; a weight kept in 32-bit gets 32-bit activations."""
    return torch.bfloat16 if compute_dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 else torch.float32
