"""RMS norm: out = w * (x * rsqrt(mean(x^2) + eps)), eps inside the root, the weight as stored
(reference: src/kernels/kernels.cpp:72-83).

A norm may be handed on *unapplied* (`deferred`): `NormedRows` names the rows, the weight and eps,
and the matrix product that consumes it applies the norm inside its own kernel when the batch is
small enough for that (decode), or asks for the rows (`materialize`) otherwise."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import TensorNeed
from .base import Norm, register_norm


class NormedRows:
    """norm(x[rows]) stored as `out_dtype`, not computed yet."""

    def __init__(self, norm: "RmsNorm", x: torch.Tensor, out_dtype: torch.dtype, rows=None):
        self.norm, self.x, self.out_dtype, self.rows = norm, x, out_dtype, rows
        self.n_rows = x.shape[0] if rows is None else rows.numel()
        self._value = None

    def materialize(self) -> torch.Tensor:
        if self._value is None:
            x = self.x
            if self.rows is not None:
                x = ops.gather_rows(self.x, self.rows, torch.empty((self.n_rows, self.x.shape[1]), dtype=torch.float32, device=self.x.device))
            self._value = self.norm(x, self.out_dtype)
        return self._value


class RmsNorm(Norm):
    graph_safe = True

    def __init__(self, spec, tensors, dtype, device):
        super().__init__(spec, tensors, dtype, device)
        self.weight = tensors[spec.weight]
        self.eps = float(spec.eps)

    @classmethod
    def tensor_needs(cls, spec):
        return [TensorNeed(spec.weight, (spec.size,), "norm")]

    def __call__(self, x, out_dtype):
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        return ops.rmsnorm(x, self.weight, self.eps, out)

    def deferred(self, x, out_dtype, rows=None) -> NormedRows:
        return NormedRows(self, x, out_dtype, rows)


register_norm("rmsnorm", RmsNorm)
