"""Causal attention with grouped key/value heads over the paged cache (optionally windowed).

Order of operations as the reference's pass (src/gpu/gpu_transformer.cpp:390-409): q, k, v
products; rotation of q and k; all new keys and values are written to their pages; then every
row attends over its request's pages up to its own position; output product added onto the
residual.  The three input products run as one with the stacked matrix [q; k; v].

The position encoding is a part of its own (`spec.position`).  One that turns the pairs
(i, i + head_dim/2) of whole heads hands over its cosines and sines, and the kernel that writes the
pages (or, for a few decoded rows, the attention kernel itself) applies them; any other encoding
changes q and k in place with its own kernels first, and the pages are then written unrotated."""
from __future__ import annotations

import torch

from ..cache.needs import PagedKvNeed
from ..kernels import ops
from ..weights.loader import TensorNeed
from .base import Mixer, PositionEncoding, position_class, register_mixer
from .linear import activation_dtype_for, linear, linear_onto
from .norm import HandedRows, NormedRows


def qkv_rotate_store_attend(h, w_qkv, ctx, cache, *, n_heads, n_kv_heads, head_dim, position=None, window=None, in_dtype=None,
                            before_rotation=None):
    """The front half of an attention-like mixer, for any mixer to call: the product with the stacked matrix [q; k; v], the
    position encoding on queries and keys, the new keys and values into the entry's pages, and every row's attention over its
    request's pages up to its own position.  Returns the heads' outputs [rows, n_heads*head_dim] in the cache's dtype.

    h                the mixer's input: rows, or a norm not yet (or half) applied, as `linear` takes it
    position         a `PositionEncoding` or None; one with `half_split_tables` is applied by the kernels that store and attend
    before_rotation  `f(q, k)`: changes the 32-bit products in place before the rotation (a norm or a scale per head; k is None
                     where the pages are another entry's).  With it the products are always written out in 32-bit; the kernels
                     that rotate, store and attend from them still serve.
    Which kernels serve is decided here by storage and shape alone: for some tens of rows and for the rows of prompts the
    product's own last step rotates and fills the pages; for a few decoded rows one kernel rotates, stores and attends;
    otherwise product, rotation + store and attention are three launches."""
    T, a_dim, kv_dim = ctx.n_rows, n_heads * head_dim, n_kv_heads * head_dim
    in_dtype = in_dtype if in_dtype is not None else activation_dtype_for(w_qkv, ctx.dtype)
    tables = position.half_split_tables(ctx) if position is not None else None
    cos, sin = tables if tables is not None else (None, None)
    att = torch.empty((T, a_dim), dtype=cache.kv.dtype, device=ctx.device)
    if (before_rotation is None and cache.writes and (tables is not None or position is None) and w_qkv.dtype == torch.bfloat16
            and cache.kv.dtype == torch.bfloat16 and in_dtype == torch.bfloat16
            and ops.gemm_bf16_qkv_rope_store_takes(T, w_qkv.shape[0], w_qkv.shape[1], head_dim)):
        # the product's own last step (the kernel that adds up the shares of k, or the epilogue over a tile) rotates and writes the pages
        # (this product finishes a norm handed on at every number of rows it is taken at, if the pieces are few enough)
        if (isinstance(h, HandedRows) and h.scaled.stride(0) % 8 == 0 and h.scaled.data_ptr() % 16 == 0
                and h.squares.shape[1] <= ops.gemm_bf16_qkv_rope_store_max_parts(T, w_qkv.shape[0], w_qkv.shape[1])):
            rows, norm_in = h.scaled, (h.squares, h.eps)
        else:
            rows, norm_in = (h.materialize() if isinstance(h, NormedRows) else h), None
        if ops.gemm_bf16_supports(rows, w_qkv, att):
            q_rot = torch.empty((T, a_dim), dtype=torch.bfloat16, device=ctx.device)
            ops.gemm_bf16_qkv_rope_store(rows, w_qkv, cos, sin, ctx.row_pos, ctx.row_slot, cache.table, q_rot, cache.kv, n_heads, n_kv_heads,
                                         head_dim, norm_in)
            return ops.attention(q_rot, cache.kv, att, ctx, cache.table, n_heads, n_kv_heads, head_dim, window)
        if norm_in is None:
            h = rows                  # (whole rows: what `linear` below would make of h)
    if cache.writes:
        qkv = torch.empty((T, a_dim + 2 * kv_dim), dtype=torch.float32, device=ctx.device)
        linear(h, w_qkv, qkv)
        q, k, v = qkv[:, :a_dim], qkv[:, a_dim:a_dim + kv_dim], qkv[:, a_dim + kv_dim:]
    else:                       # the pages are another layer's: only the queries are made
        q, k, v = torch.empty((T, a_dim), dtype=torch.float32, device=ctx.device), None, None
        linear(h, w_qkv[:a_dim], q)
    if before_rotation is not None:
        before_rotation(q, k)
    if position is not None and tables is None:          # an encoding with kernels of its own: q and k are turned in place
        position.apply(q, k, ctx, n_heads, n_kv_heads, head_dim)
    # a step of single decoded rows: one kernel rotates, writes the pages and attends
    if not ops.attention_from_products(q, k, v, cos, sin, cache.kv, att, ctx, cache.table, n_heads, n_kv_heads, head_dim, window):
        q_rot = torch.empty((T, a_dim), dtype=cache.kv.dtype, device=ctx.device)
        ops.rope_store(q, k, v, cos, sin, ctx.row_pos, ctx.row_slot, cache.table, q_rot, cache.kv, n_heads, n_kv_heads, head_dim)
        ops.attention(q_rot, cache.kv, att, ctx, cache.table, n_heads, n_kv_heads, head_dim, window)
    return att


class Attention(Mixer):
    accepts_deferred_norm = True      # its input goes into `linear` only
    hands_norm_on = True              # `forward` takes `then`, the norm that reads the residual next

    def __init__(self, spec, tensors, dtype, device):
        super().__init__(spec, tensors, dtype, device)
        s = spec
        if s.n_heads % s.n_kv_heads:
            raise ValueError("the number of heads must be a multiple of the number of key/value heads")
        if not 0 < s.head_dim <= ops.attention_max_head_size():
            raise ValueError(f"attention: head_dim = {s.head_dim} is outside what the attention kernels take (1 to {ops.attention_max_head_size()} channels a head)")
        self.a_dim, self.kv_dim = s.n_heads * s.head_dim, s.n_kv_heads * s.head_dim
        self.w_qkv = torch.cat([tensors[s.q_proj], tensors[s.k_proj], tensors[s.v_proj]], dim=0).contiguous()
        self.w_o = tensors[s.o_proj]
        self.position = None if s.position is None else position_class(s.position)(s.position, tensors, dtype, device)
        self.in_dtype = activation_dtype_for(self.w_qkv, dtype)
        self.att_dtype = activation_dtype_for(self.w_o, dtype)
        self.graph_safe = self.position is None or bool(getattr(self.position, "graph_safe", False))

    @classmethod
    def tensor_needs(cls, spec):
        a, kv, d = spec.n_heads * spec.head_dim, spec.n_kv_heads * spec.head_dim, spec.hidden_size
        return [TensorNeed(spec.q_proj, (a, d)), TensorNeed(spec.k_proj, (kv, d)), TensorNeed(spec.v_proj, (kv, d)),
                TensorNeed(spec.o_proj, (d, a))]

    @classmethod
    def cache_need(cls, spec):
        return PagedKvNeed(spec.n_kv_heads, spec.head_dim, spec.window)

    def takes_handed_norm(self, n_rows: int) -> bool:
        if self.in_dtype != torch.bfloat16:
            return False
        if ops.gemm_bf16_takes_norm(n_rows, self.w_qkv.shape[0], self.w_qkv.shape[1]):
            return True
        # the rows of prompts: the q/k/v product that rotates and fills the pages itself finishes the norm, where it serves
        half_split = self.position is None or getattr(type(self.position), "half_split_tables", None) is not PositionEncoding.half_split_tables
        return half_split and ops.gemm_bf16_qkv_rope_store_takes(n_rows, self.w_qkv.shape[0], self.w_qkv.shape[1], self.spec.head_dim)

    def forward(self, h, residual, ctx, cache, then=None):
        s = self.spec
        att = qkv_rotate_store_attend(h, self.w_qkv, ctx, cache, n_heads=s.n_heads, n_kv_heads=s.n_kv_heads, head_dim=s.head_dim,
                                      position=self.position, window=s.window, in_dtype=self.in_dtype)
        if att.dtype != self.att_dtype:
            att = att.to(self.att_dtype)
        return linear_onto(att, self.w_o, residual, then)


register_mixer("attention", Attention)
