"""Arrangements of a layer's parts around the residual stream.

"prenorm" (reference: src/model/transformer.cpp:385-450):
    x += mixer(norm_1(x));  x += feed_forward(norm_2(x))
The residual stream x is float32 [T, hidden] and is changed in place."""
from __future__ import annotations

from .base import feed_forward_class, mixer_class, norm_class, register_block
from .norm import norm_to_hand_on


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

    # A part that adds onto the residual may do the next norm's share on the way (`HandedRows` in parts/norm.py), if that
    # norm can be applied so (`handed_weight`), its reader takes rows so normed (`takes_handed_norm`) and the part knows how
    # (`hands_norm_on`: its `forward` takes `then` and returns the handed rows, or None where its product could not).
    hands_norm_on = True

    def first_reader(self):
        """The norm that reads the residual first in this block, and the part that reads the normed rows."""
        return self.mixer_norm, self.mixer

    @staticmethod
    def _then(part, reader, n_rows):
        return norm_to_hand_on(reader, n_rows) if getattr(part, "hands_norm_on", False) else None

    def forward(self, x, ctx, cache, handed=None, next_reader=None):
        """handed: this block's first norm as whoever wrote x last left it, or None.  next_reader: `first_reader()` of whatever
        reads x after this block, or None.  Returns that reader's norm handed on, or None."""
        if handed is None or handed.norm is not self.mixer_norm:
            handed = self._normed(self.mixer_norm, self.mixer, x, ctx)
        then = self._then(self.mixer, (self.feed_forward_norm, self.feed_forward), ctx.n_rows)
        handed = self.mixer.forward(handed, x, ctx, cache) if then is None else self.mixer.forward(handed, x, ctx, cache, then=then)
        if ctx.trace is not None:
            ctx.trace("attn_out", x)
        if handed is None or then is None:
            handed = self._normed(self.feed_forward_norm, self.feed_forward, x, ctx)
        then = self._then(self.feed_forward, next_reader, ctx.n_rows)
        handed = self.feed_forward.forward(handed, x, ctx) if then is None else self.feed_forward.forward(handed, x, ctx, then=then)
        if ctx.trace is not None:
            ctx.trace("ffn_out", x)
        return handed if then is not None else None


register_block("prenorm", PreNormBlock)
