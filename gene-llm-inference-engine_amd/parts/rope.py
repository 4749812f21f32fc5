"""Rotary position encoding with half-split pairs.

Frequencies are computed once, in 64-bit on the host, as the reference computes them
(src/kernels/kernels.cpp:142-147): f_k = theta^(-2k/head_dim), unless the spec brings the
frequencies an architecture's own rule has made of them.  Per step, cos and sin of pos*f_k are
made on the device from 64-bit angles for the step's rows and shared by every layer with the
same spec."""
from __future__ import annotations

import math

import torch

from ..kernels import ops
from .base import PositionEncoding, register_position_encoding

def inverse_frequencies(head_dim: int, theta: float):
    return [1.0 / math.pow(float(theta), 2.0 * k / head_dim) for k in range(head_dim // 2)]


class RotaryHalfSplit(PositionEncoding):
    graph_safe = True

    def __init__(self, spec, tensors, dtype, device):
        super().__init__(spec, tensors, dtype, device)
        if spec.head_dim % 2:
            raise ValueError("rotary encoding needs an even head size")
        self.half = spec.head_dim // 2
        frequencies = spec.frequencies if spec.frequencies is not None else inverse_frequencies(spec.head_dim, spec.theta)
        self.inv_freq = torch.tensor(list(frequencies), dtype=torch.float64, device=device)

    def half_split_tables(self, ctx):
        """(cos, sin), float32 [T, head_dim/2], for the rows of this step."""
        key = ("rotary", self.spec)
        if key not in ctx.memo:
            cos = torch.empty((ctx.n_rows, self.half), dtype=torch.float32, device=ctx.device)
            sin = torch.empty_like(cos)
            ops.rope_cos_sin(ctx.row_pos, self.inv_freq, cos, sin)
            ctx.memo[key] = (cos, sin)
        return ctx.memo[key]


register_position_encoding("rotary_half_split", RotaryHalfSplit)
