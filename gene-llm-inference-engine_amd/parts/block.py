"""Arrangements of a layer's parts around the residual stream.

"prenorm" (reference: src/model/transformer.cpp:385-450):
    x += mixer(norm_1(x));  x += feed_forward(norm_2(x))
The residual stream x is float32 [T, hidden] and is changed in place."""
from __future__ import annotations

from .base import feed_forward_class, mixer_class, norm_class, register_block


class PreNormBlock:
    def __init__(self, spec, tensors, dtype, device):
        self.spec = spec
        self.mixer_norm = norm_class(spec.mixer_norm)(spec.mixer_norm, tensors, dtype, device)
        self.mixer = mixer_class(spec.mixer)(spec.mixer, tensors, dtype, device)
        self.feed_forward_norm = norm_class(spec.feed_forward_norm)(spec.feed_forward_norm, tensors, dtype, device)
        self.feed_forward = feed_forward_class(spec.feed_forward)(spec.feed_forward, tensors, dtype, device)

    @property
    def graph_safe(self):
        return all(getattr(p, "graph_safe", False) for p in (self.mixer_norm, self.mixer, self.feed_forward_norm, self.feed_forward))

    @classmethod
    def tensor_needs(cls, spec):
        return (norm_class(spec.mixer_norm).tensor_needs(spec.mixer_norm) + mixer_class(spec.mixer).tensor_needs(spec.mixer) +
                norm_class(spec.feed_forward_norm).tensor_needs(spec.feed_forward_norm) +
                feed_forward_class(spec.feed_forward).tensor_needs(spec.feed_forward))

    @classmethod
    def cache_need(cls, spec):
        return mixer_class(spec.mixer).cache_need(spec.mixer)

    @staticmethod
    def _normed(norm, part, x, ctx):
        """The part's input: the normed rows, or the norm handed on unapplied if both sides can."""
        dtype = getattr(part, "in_dtype", ctx.dtype)
        if getattr(part, "accepts_deferred_norm", False) and hasattr(norm, "deferred"):
            return norm.deferred(x, dtype)
        return norm(x, dtype)

    def forward(self, x, ctx, cache):
        self.mixer.forward(self._normed(self.mixer_norm, self.mixer, x, ctx), x, ctx, cache)
        if ctx.trace is not None:
            ctx.trace("attn_out", x)
        self.feed_forward.forward(self._normed(self.feed_forward_norm, self.feed_forward, x, ctx), x, ctx)
        if ctx.trace is not None:
            ctx.trace("ffn_out", x)


register_block("prenorm", PreNormBlock)
