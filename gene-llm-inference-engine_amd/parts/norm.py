"""RMS norm: out = w * (x * rsqrt(mean(x^2) + eps)), eps inside the root, the weight as stored
(reference: src/kernels/kernels.cpp:72-83).

A norm may be handed on *unapplied* (`deferred`): `NormedRows` names the rows (optionally a
selection of them), the weight and eps; whoever consumes it asks for the rows (`materialize`), and
the norm's kernel gathers the selection itself.

A norm may also be *half applied* by the product that wrote the rows last (`HandedRows`): that
product, when it adds onto the rows x, also writes w * x in bfloat16 and the pieces of every row's
sum of squares, and the product that reads the normed rows multiplies its results by
rsqrt(mean(x^2) + eps), which is one number a row and commutes with it.  For a few rows (decoding)
this saves the norm's kernel; `linear` decides where it applies, and `materialize` still gives the
rows the ordinary way."""
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
            self._value = self.norm(self.x, self.out_dtype, self.rows)
        return self._value


class HandedRows(NormedRows):
    """norm(x) as bfloat16, half applied: `scaled` = w * x, `squares` [rows, pieces] = the pieces of the rows' sums of x^2."""

    def __init__(self, norm: "RmsNorm", x: torch.Tensor, scaled: torch.Tensor, squares: torch.Tensor):
        super().__init__(norm, x, torch.bfloat16)
        self.scaled, self.squares, self.eps = scaled, squares, norm.eps


def norm_to_hand_on(reader, n_rows: int):
    """reader: (norm, part) as a block's `first_reader()` gives it, or None.  The norm, if whoever writes the rows it reads
    next can apply it half way (`HandedRows`): it has weights to apply so (`handed_weight`) and the part's first product
    finishes such a norm at this number of rows (`accepts_deferred_norm`, `takes_handed_norm`); None otherwise."""
    norm, part = reader if reader is not None else (None, None)
    if (norm is None or not hasattr(norm, "handed_weight") or not getattr(part, "accepts_deferred_norm", False)
            or not hasattr(part, "takes_handed_norm") or not part.takes_handed_norm(n_rows)):
        return None
    return norm


class RmsNorm(Norm):
    graph_safe = True

    def __init__(self, spec, tensors, dtype, device):
        super().__init__(spec, tensors, dtype, device)
        self.weight = tensors[spec.weight]
        self.eps = float(spec.eps)
        # the weights once more in 32-bit, for a product that applies them to rows it has just written (`handed_weight`); made
        # here, not at first use, which might fall into the capture of a graph
        self._handed_weight = self.weight if self.weight.dtype == torch.float32 else self.weight.float().contiguous()

    @classmethod
    def tensor_needs(cls, spec):
        return [TensorNeed(spec.weight, (spec.size,), "norm")]

    def __call__(self, x, out_dtype, rows=None):
        """The normed rows of x, or of x[rows]."""
        n = x.shape[0] if rows is None else rows.numel()
        out = torch.empty((n, x.shape[1]), dtype=out_dtype, device=x.device)
        if rows is not None and not ops.rmsnorm_can_gather(x, self.weight, out):
            x, rows = ops.gather_rows(x, rows, torch.empty((n, x.shape[1]), dtype=torch.float32, device=x.device)), None
        return ops.rmsnorm(x, self.weight, self.eps, out, rows)

    def deferred(self, x, out_dtype, rows=None) -> NormedRows:
        return NormedRows(self, x, out_dtype, rows)

    def handed_weight(self) -> torch.Tensor:
        """The weights in 32-bit, for a product that applies them to the rows it has just written."""
        return self._handed_weight

    def weights_read_per_step(self):
        """One copy of the weights: a step reads them as stored (the norm's kernel) or in 32-bit (a product that does the
        norm's share), never both."""
        return [self.weight]


register_norm("rmsnorm", RmsNorm)
