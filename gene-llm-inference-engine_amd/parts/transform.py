"""Elementwise changes of float32 rows in place, for the two places a model may ask for one: between the token
table and the first layer (`ModelSpec.after_embedding`) and on the logits (`ModelSpec.after_head`)."""
from __future__ import annotations

from ..kernels import ops
from .base import RowTransform, register_row_transform


class ScaleRows(RowTransform):
    graph_safe = True

    def __call__(self, x):
        ops.scale_rows(x, float(self.spec.factor))


class SoftCap(RowTransform):
    graph_safe = True

    def __call__(self, x):
        ops.softcap_rows(x, float(self.spec.cap))


register_row_transform("scale", ScaleRows)
register_row_transform("softcap", SoftCap)
