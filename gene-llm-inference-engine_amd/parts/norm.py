"""RMS norm: out = w * (x * rsqrt(mean(x^2) + eps)), eps inside the root, the weight as stored
(reference: src/kernels/kernels.cpp:72-83)."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import TensorNeed
from .base import Norm, register_norm


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


register_norm("rmsnorm", RmsNorm)
