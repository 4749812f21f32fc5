"""Rotary position encoding with half-split pairs and the optional llama3 change of frequencies.

Frequencies are computed once, in 64-bit on the host, as the reference computes them per
frequency (src/kernels/kernels.cpp:142-158): f_k = theta^(-2k/head_dim); with scaling, a
wavelength 2*pi/f above original/low_freq_factor divides f by `factor`, one below
original/high_freq_factor leaves it, and between the two f is blended.  Per step, cos and sin
of pos*f_k are made on the device from 64-bit angles for the step's rows and shared by every
layer with the same spec."""
from __future__ import annotations

import math

import torch

from ..kernels import ops
from .base import PositionEncoding, register_position_encoding

_TWO_PI = 6.283185307179586476925


def inverse_frequencies(head_dim: int, theta: float, scaling=None):
    out = []
    for k in range(head_dim // 2):
        f = 1.0 / math.pow(float(theta), 2.0 * k / head_dim)
        if scaling is not None:
            wavelength = _TWO_PI / f
            original = float(scaling.original_max_position_embeddings)
            if wavelength > original / scaling.low_freq_factor:
                f /= scaling.factor
            elif not wavelength < original / scaling.high_freq_factor:
                smooth = (original / wavelength - scaling.low_freq_factor) / (scaling.high_freq_factor - scaling.low_freq_factor)
                f = (1.0 - smooth) * f / scaling.factor + smooth * f
        out.append(f)
    return out


class RotaryHalfSplit(PositionEncoding):
    graph_safe = True

    def __init__(self, spec, tensors, dtype, device):
        super().__init__(spec, tensors, dtype, device)
        if spec.head_dim % 2:
            raise ValueError("rotary encoding needs an even head size")
        self.half = spec.head_dim // 2
        self.inv_freq = torch.tensor(inverse_frequencies(spec.head_dim, spec.theta, spec.scaling), dtype=torch.float64, device=device)

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
