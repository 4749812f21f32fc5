"""SwiGLU feed-forward: residual += down( silu(gate(h)) * up(h) ), silu(g) = g / (1 + exp(-g))
(reference: src/model/transformer.cpp:437-450).  gate and up run as one product with the stacked
matrix [gate; up]."""
from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.loader import TensorNeed
from .base import FeedForward, register_feed_forward
from .linear import activation_dtype_for, linear, linear_onto


class SwiGlu(FeedForward):
    graph_safe = True
    accepts_deferred_norm = True      # its input goes into `linear` only
    hands_norm_on = True              # `forward` takes `then`, the norm that reads the residual next

    def __init__(self, spec, tensors, dtype, device):
        super().__init__(spec, tensors, dtype, device)
        gate, up = tensors[spec.gate_proj], tensors[spec.up_proj]
        self.w_down = tensors[spec.down_proj]
        self.in_dtype = activation_dtype_for(gate, dtype)
        self.mid_dtype = activation_dtype_for(self.w_down, dtype)
        # bfloat16 throughout: the gate is applied inside the product (weights interleaved for it)
        self.fused = (self.in_dtype == torch.bfloat16 and self.mid_dtype == torch.bfloat16 and up.dtype == torch.bfloat16
                      and spec.intermediate_size % 16 == 0 and spec.hidden_size % 8 == 0)
        self.w_gate_up = ops.interleave_gate_up(gate, up) if self.fused else torch.cat([gate, up], dim=0).contiguous()

    @classmethod
    def tensor_needs(cls, spec):
        i, d = spec.intermediate_size, spec.hidden_size
        return [TensorNeed(spec.gate_proj, (i, d)), TensorNeed(spec.up_proj, (i, d)), TensorNeed(spec.down_proj, (d, i))]

    def takes_handed_norm(self, n_rows: int) -> bool:
        return self.in_dtype == torch.bfloat16 and ops.gemm_bf16_takes_norm(n_rows, self.w_gate_up.shape[0], self.w_gate_up.shape[1], self.fused)

    def forward(self, h, residual, ctx, then=None):
        T, inter = ctx.n_rows, self.spec.intermediate_size
        if self.fused:
            mid = torch.empty((T, inter), dtype=torch.bfloat16, device=ctx.device)
            linear(h, self.w_gate_up, mid, gated=True)
            return linear_onto(mid, self.w_down, residual, then)
        gate_up = torch.empty((T, 2 * inter), dtype=torch.float32, device=ctx.device)
        linear(h, self.w_gate_up, gate_up)
        mid = torch.empty((T, inter), dtype=self.mid_dtype, device=ctx.device)
        ops.silu_mul(gate_up, mid)
        return linear_onto(mid, self.w_down, residual, then)


register_feed_forward("swiglu", SwiGlu)
