"""A decoder assembled from a `ModelSpec`: token table, the layers in their run order, final
norm, output head.  It knows parts and the order they run in, not an architecture."""
from __future__ import annotations

from pathlib import Path
from typing import Dict, List, Optional

import torch

from ..config import ModelSpec, read_config
from ..kernels import ops
from ..parts import LayerCache, StepContext, block_class, linear, model_tensor_needs, norm_class, row_transform_class, weight_bytes
from ..parts.linear import activation_dtype_for
from ..parts.norm import HandedRows, norm_to_hand_on
from ..weights import load_tensors, random_tensors

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32,
           torch.bfloat16: torch.bfloat16, torch.float32: torch.float32}


def compute_dtype(name) -> torch.dtype:
    try:
        return _DTYPES[name]
    except KeyError:
        raise ValueError(f"unknown dtype {name!r}: bfloat16 or float32") from None


class _Head:
    """The output head as the reader of the final norm: asked, like a part, whether it takes that norm half applied."""
    accepts_deferred_norm = True

    def __init__(self, weight: torch.Tensor, in_dtype: torch.dtype):
        self.weight, self.in_dtype = weight, in_dtype

    def takes_handed_norm(self, n_rows: int) -> bool:
        return self.in_dtype == torch.bfloat16 and ops.gemm_bf16_takes_norm(n_rows, self.weight.shape[0], self.weight.shape[1])


class DecoderModel:
    def __init__(self, spec: ModelSpec, tensors: Dict[str, torch.Tensor], dtype: torch.dtype, device):
        self.spec, self.dtype, self.device = spec, dtype, torch.device(device)
        self.embedding = tensors[spec.embedding]
        self.lm_head = tensors[spec.lm_head]
        self.layers = [block_class(l.block)(l, tensors, dtype, device) for l in spec.layers]
        self.final_norm = norm_class(spec.final_norm)(spec.final_norm, tensors, dtype, device)
        self.head_in_dtype = activation_dtype_for(self.lm_head, dtype)
        self.head = _Head(self.lm_head, self.head_in_dtype)
        self.after_embedding = [row_transform_class(t)(t, tensors, dtype, device) for t in spec.after_embedding]
        self.after_head = [row_transform_class(t)(t, tensors, dtype, device) for t in spec.after_head]
        self.run_order = spec.run_order
        self.trace = None                        # see set_trace
        self.graph_safe = all(getattr(p, "graph_safe", False) for p in (*self.layers, self.final_norm, *self.after_embedding, *self.after_head))

    # ----------------------------------------------------------------------------- what it needs
    def cache_needs(self):
        """Per run-order entry: its cache need, and the entry whose cache it reads (or None)."""
        needs = [block_class(self.spec.layers[e.layer].block).cache_need(self.spec.layers[e.layer]) for e in self.run_order]
        return needs, [e.cache_of for e in self.run_order]

    def weight_bytes_read_per_step(self) -> int:
        """Bytes of weights one step reads when it uses every matrix once: what every part of the run order holds (a
        layer named twice is read twice), the final norm and the head; the token table is read by row and not counted."""
        return (sum(weight_bytes(self.layers[e.layer]) for e in self.run_order) + weight_bytes(self.final_norm) + weight_bytes(self.lm_head)
                + weight_bytes(self.after_embedding) + weight_bytes(self.after_head))

    # ------------------------------------------------------------------------------- the pass
    def forward(self, ctx: StepContext, cache, logit_rows: Optional[torch.Tensor], n_logit_rows: int):
        """Runs the step's rows through every layer of the run order; returns float32 logits
        [n_logit_rows, vocab] of the rows listed in `logit_rows`, or None if there are none."""
        x = torch.empty((ctx.n_rows, self.spec.hidden_size), dtype=torch.float32, device=self.device)
        trace = self.trace
        handed = self._embed(ctx, x)      # the next block's first norm, where whoever wrote x could leave it half applied
        if trace is not None:
            trace("embedding", -1, x)
        for i, entry in enumerate(self.run_order):
            ctx.trace = None if trace is None else (lambda tag, rows, i=i: trace(tag, i, rows))
            layer = self.layers[entry.layer]
            if getattr(layer, "hands_norm_on", False):
                if i + 1 < len(self.run_order):
                    after = self.layers[self.run_order[i + 1].layer]
                    reader = after.first_reader() if getattr(after, "hands_norm_on", False) else None
                else:                     # the head reads every row of the final norm, or a selection, which is not handed on
                    reader = (self.final_norm, self.head) if ctx.every_row_wanted and trace is None else None
                handed = layer.forward(x, ctx, cache.layer_cache(i), handed=handed, next_reader=reader)
            else:
                layer.forward(x, ctx, cache.layer_cache(i))
                handed = None
        ctx.trace = None
        if n_logit_rows == 0:
            return None
        logits = torch.empty((n_logit_rows, self.spec.vocab_size), dtype=torch.float32, device=self.device)
        if handed is not None and handed.norm is self.final_norm and ctx.every_row_wanted:
            normed = handed
        elif hasattr(self.final_norm, "deferred"):
            normed = self.final_norm.deferred(x, self.head_in_dtype, rows=logit_rows)
        else:
            picked = torch.empty((n_logit_rows, self.spec.hidden_size), dtype=torch.float32, device=self.device)
            normed = self.final_norm(ops.gather_rows(x, logit_rows, picked), self.head_in_dtype)
        if trace is not None:
            trace("final_norm", -1, normed if torch.is_tensor(normed) else self.final_norm(ops.gather_rows(x, logit_rows, torch.empty(
                (n_logit_rows, self.spec.hidden_size), dtype=torch.float32, device=self.device)), torch.float32))
        linear(normed, self.lm_head, logits)
        for transform in self.after_head:
            transform(logits)
        return logits

    def _embed(self, ctx: StepContext, x: torch.Tensor):
        """The rows of the token table into x.  Where the first block's first norm can be taken half applied (`HandedRows`: a few
        single rows of decoding requests in bfloat16, a norm of the form g * x * rsqrt(mean square + eps), a reader whose product
        finishes it), the kernel that fetches the rows does the norm's first half too and the `HandedRows` are returned; None otherwise."""
        first = self.layers[self.run_order[0].layer] if self.run_order else None
        if (first is not None and not self.after_embedding and self.trace is None and self.dtype == torch.bfloat16
                and getattr(first, "hands_norm_on", False) and ctx.max_seg_len == 1):         # (decode steps: the one norm kernel of a step that is all launches)
            norm = norm_to_hand_on(first.first_reader(), ctx.n_rows)
            if norm is not None:
                scaled = torch.empty((ctx.n_rows, self.spec.hidden_size), dtype=torch.bfloat16, device=self.device)
                squares = torch.empty((ctx.n_rows, 1), dtype=torch.float32, device=self.device)
                ops.embed_handing(self.embedding, ctx.tokens, x, norm.handed_weight(), scaled, squares)
                return HandedRows(norm, x, scaled, squares)
        ops.embed(self.embedding, ctx.tokens, x)
        for transform in self.after_embedding:
            transform(x)
        return None

    def set_trace(self, trace) -> None:
        """Debugging, as the reference's Model::set_trace (src/model/model.h): `trace(tag, run-order entry or -1, rows)` is
        called with the step's residual stream after the embedding ("embedding"), after each half of every block
        ("attn_out", "ffn_out") and with the normed rows that the logits are taken from ("final_norm").  While a trace is
        set no step is replayed from a captured graph."""
        self.trace = trace


def load_model(folder, dtype="bfloat16", device="cuda:0") -> DecoderModel:
    """The model a folder (config.json, model.safetensors) describes; the class of its
    configuration is chosen by config.json."""
    dtype = compute_dtype(dtype)
    config = read_config(folder)
    spec = config.model_spec()
    tensors = load_tensors(folder, model_tensor_needs(spec), dtype, device, spec.ignorable_tensors)
    model = DecoderModel(spec, tensors, dtype, device)
    model.config = config
    return model


def random_model(config, seed: int, dtype="bfloat16", device="cuda:0", std: float = 0.02, draw_on_device: bool = False) -> DecoderModel:
    """A model of `config` with seeded random weights, without a folder in between.  With
    `draw_on_device` the numbers are made on the device by a formula of (seed, tensor name, element index)
    (`weights.random_init`: fast for large models, and anybody can re-make them; other numbers than the
    host generator gives for the same seed)."""
    dtype = compute_dtype(dtype)
    spec = config.model_spec()
    if draw_on_device:
        from ..weights import formula_tensors
        tensors = formula_tensors(model_tensor_needs(spec), seed, dtype, std, device)
    else:
        host = random_tensors(model_tensor_needs(spec), seed, dtype, std)
        tensors = {k: v.to(device) for k, v in host.items()}
    model = DecoderModel(spec, tensors, dtype, device)
    model.config = config
    return model
