"""Interfaces of the parts a layer is put together from, and the registries that map a spec's
`kind` to the class that implements it.

A part is built from its spec (all sizes and constants), the weight tensors it named, the compute
dtype and the device.  It never sees the model it is in.  During a step it gets a `StepContext`
(what the batch looks like) and, if it keeps a cache, a `LayerCache` (its own view of the cache
manager).

Kinds of parts and what each must provide:

* norm:              `tensor_needs(spec)`, `__call__(x_f32[T, size], out_dtype) -> [T, size]`
* position encoding: `apply(q, k, ctx, ...)` turns the float32 queries and keys of a step's rows in place, with
                     kernels of its own; or `half_split_tables(ctx) -> (cos, sin)` if it is a rotation of the pairs
                     (i, i + head_dim/2) of whole heads, which the attention kernels apply themselves
* row transform:     `__call__(x_f32[T, n])` changes rows in place (after the embedding, or on the logits)
* mixer:             `tensor_needs(spec)`, `cache_need(spec)`, `forward(h, residual, ctx, cache)`
* feed-forward:      `tensor_needs(spec)`, `forward(h, residual, ctx)`
* block:             `forward(x, ctx, cache)` wiring norms, mixer and feed-forward around the
                     32-bit residual stream `x`

Mixers and feed-forwards add their result onto `residual` (float32 [T, hidden]) in place.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable, Dict, List, Optional

import numpy as np
import torch

from ..weights.loader import TensorNeed


@dataclass
class StepContext:
    """One step's batch as the parts see it.  Rows are the tokens of the step in the order given;
    the rows of one request are consecutive and in position order."""
    n_rows: int
    dtype: torch.dtype                       # compute dtype: what activations between parts are stored as
    device: torch.device
    tokens: torch.Tensor                     # int32 [T]
    row_pos: torch.Tensor                    # int32 [T]  position of each row in its request
    row_slot: torch.Tensor                   # int32 [T]  the request's slot (row of page tables and state tensors)
    seg_slot: List[int]                      # per request of the step, on the host: slot,
    seg_start: List[int]                     # first row,
    seg_len: List[int]                       # number of rows,
    seg_pos0: List[int]                      # position of the first row
    memo: Dict[Any, Any] = field(default_factory=dict)     # per-step tables shared by layers (rotary cos/sin)
    upload: Optional[Callable[..., Any]] = None    # the runner's way of bringing int32 step data to the device: upload(a) -> tensor, upload(a, b) -> (tensor, tensor) in one copy
    trace: Optional[Callable[[str, torch.Tensor], None]] = None        # debugging: a block reports (tag, residual stream [T, hidden]) after each of its two halves
    every_row_wanted: bool = False           # the step's logits are asked for at every row, in the rows' order

    def to_device(self, *values):
        """int32 data made on the host for this step (row lists, tile lists) as device tensors, valid during the step:
        one tensor for one list, a tuple for several (which the runner sends in one copy)."""
        arrays = [np.ascontiguousarray(v, dtype=np.int32) for v in values]
        if self.upload is not None:
            return self.upload(*arrays)
        pieces = tuple(torch.from_numpy(a).to(self.device) for a in arrays)
        return pieces[0] if len(pieces) == 1 else pieces

    @property
    def max_seg_len(self) -> int:
        return max(self.seg_len)

    @property
    def max_context(self) -> int:
        return max(p + n for p, n in zip(self.seg_pos0, self.seg_len))


@dataclass
class LayerCache:
    """A run-order entry's view of the cache manager."""
    kv: Optional[torch.Tensor] = None        # [page, 2, kv_head, place, head_dim] of this layer
    table: Optional[torch.Tensor] = None     # int32 [slot, pages]
    state: Optional[torch.Tensor] = None     # [slot, ...] fixed-size state
    writes: bool = True                      # False: the pages belong to another entry, read only


class Part:
    """Common construction: `spec`, `tensors` (by name, on the device), compute dtype, device.

    `graph_safe` says that everything in the part's work that changes from step to step is read on
    the device (from the context's tensors, the page tables, the cache and the state slots), never from
    the context's host-side lists, and that no shape depends on the data: only then may a step be
    captured once and replayed.  What a captured pass may take from the host is its shape, which every
    replay shares: the number of rows, where each request's rows begin and how many they are
    (`seg_start`, `seg_len`); not the requests' slots or positions (`seg_slot`, `seg_pos0`: on the
    device they are `row_slot` and `row_pos`).  It is False unless a part says otherwise, and one
    part that is not makes the runner launch every step anew."""
    graph_safe = False

    def __init__(self, spec, tensors: Dict[str, torch.Tensor], dtype: torch.dtype, device):
        self.spec, self.dtype, self.device = spec, dtype, device

    @classmethod
    def tensor_needs(cls, spec) -> List[TensorNeed]:
        return []


class Mixer(Part):
    """A mixer with a `StateNeed` takes the rows of a request in order, reads `cache.state[slot]` at the first and may
    write it as it goes: the step function puts the slots of a step's requests back as they were if the pass raises."""

    @classmethod
    def cache_need(cls, spec):
        """A `PagedKvNeed`, a `StateNeed` or None."""
        return None

    def forward(self, h: torch.Tensor, residual: torch.Tensor, ctx: StepContext, cache: LayerCache) -> None:
        raise NotImplementedError


class FeedForward(Part):
    def forward(self, h: torch.Tensor, residual: torch.Tensor, ctx: StepContext) -> None:
        raise NotImplementedError


# Optional, for a mixer or feed-forward (none of it is needed; a part without it is served the ordinary way):
#   accepts_deferred_norm = True   `h` may be a norm not yet applied (parts/norm.py: `NormedRows`), which the part passes to `linear`
#                                  unchanged; it may then also be a norm half applied by whoever wrote the rows (`HandedRows`), if
#   takes_handed_norm(n_rows)      says that the part's first product can finish such a norm at this number of rows.
#   hands_norm_on = True           `forward` takes a keyword `then`, the norm that will read `residual` next, adds onto the residual with
#                                  `linear_onto(..., then)` and returns what that returns (the `HandedRows`, or None).


# Optional, for a block (an arrangement of parts; of however many halves):
#   hands_norm_on = True           the block plays the same game towards its neighbours in the run order: `first_reader()` returns the
#                                  norm that reads the residual first in it and the part that reads the normed rows, and `forward`
#                                  takes the keywords `handed` (that norm as whoever wrote the residual last left it, `HandedRows` or
#                                  None) and `next_reader` (`first_reader()` of whatever reads the residual after the block, or None)
#                                  and returns that reader's norm handed on, or None.  The model only carries these between the blocks
#                                  (and plays the first writer and the last reader itself: the token rows, the final norm and the
#                                  head); `norm_to_hand_on` in parts/norm.py is the one test of whether a reader can take it.


class Norm(Part):
    def __call__(self, x: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
        raise NotImplementedError


class PositionEncoding(Part):
    """How positions enter a mixer's queries and keys.  A mixer asks `half_split_tables` first: an encoding that
    turns the pairs (i, i + head_dim/2) of every whole head by an angle per (row, pair) answers with the angles'
    cosines and sines, and the kernels that write the cache and attend apply them on the way (nothing is launched
    for the rotation).  Every other encoding (another pairing, a part of the head only, something that is no
    rotation) answers None and gets `apply` called with the rows' float32 queries and keys, which it changes in
    place with kernels of its own before they are stored and attended over."""

    def half_split_tables(self, ctx: StepContext):
        """(cos, sin), float32 [rows, head_dim/2] each, made once per step (kept in ctx.memo), or None."""
        return None

    def apply(self, q: torch.Tensor, k: Optional[torch.Tensor], ctx: StepContext, n_heads: int, n_kv_heads: int, head_dim: int) -> None:
        """q: float32 [rows, n_heads*head_dim], k: float32 [rows, n_kv_heads*head_dim] or None (the keys are another
        entry's); both may be column ranges of a wider tensor (unit inner stride, any row stride)."""
        raise NotImplementedError(f"{type(self).__name__} gives neither half-split tables nor an apply step")


class RowTransform(Part):
    """An elementwise change of float32 rows in place: what a model may ask for between the token table and the
    first layer, and on the logits."""

    def __call__(self, x: torch.Tensor) -> None:
        raise NotImplementedError


def weight_tensors(obj, _seen=None):
    """The floating-point tensors that `obj` (a part, a block, a list of them) holds, each object visited once:
    what a step reads of it when it uses every weight once.  A part whose step reads other tensors than it holds
    (experts of which only some run) says which in a method `weights_read_per_step()`."""
    seen = _seen if _seen is not None else set()
    if id(obj) in seen:
        return
    seen.add(id(obj))
    if torch.is_tensor(obj):
        if obj.dtype in (torch.bfloat16, torch.float32, torch.float16):
            yield obj
    elif isinstance(obj, (list, tuple)):
        for v in obj:
            yield from weight_tensors(v, seen)
    elif isinstance(obj, dict):
        for v in obj.values():
            yield from weight_tensors(v, seen)
    elif callable(getattr(obj, "weights_read_per_step", None)):
        yield from weight_tensors(list(obj.weights_read_per_step()), seen)
    elif isinstance(obj, Part) or callable(getattr(obj, "forward", None)):
        for v in vars(obj).values():
            yield from weight_tensors(v, seen)


def weight_bytes(obj) -> int:
    """Bytes of `weight_tensors(obj)`, memory that several of them name counted once."""
    by_address: Dict[int, int] = {}
    for t in weight_tensors(obj):
        by_address[t.data_ptr()] = max(by_address.get(t.data_ptr(), 0), t.numel() * t.element_size())
    return sum(by_address.values())


_REGISTRIES: Dict[str, Dict[str, type]] = {"mixer": {}, "feed_forward": {}, "norm": {}, "position": {}, "block": {}, "row_transform": {}}


def _register(family: str, kind: str, cls: type) -> None:
    table = _REGISTRIES[family]
    if kind in table and table[kind] is not cls:
        raise ValueError(f"{family} kind '{kind}' is already registered")
    table[kind] = cls


def _lookup(family: str, kind: str) -> type:
    try:
        return _REGISTRIES[family][kind]
    except KeyError:
        raise KeyError(f"no {family} of kind '{kind}' is registered; known: {', '.join(sorted(_REGISTRIES[family]))}") from None


def register_mixer(kind, cls): _register("mixer", kind, cls)
def register_feed_forward(kind, cls): _register("feed_forward", kind, cls)
def register_norm(kind, cls): _register("norm", kind, cls)
def register_position_encoding(kind, cls): _register("position", kind, cls)
def register_block(kind, cls): _register("block", kind, cls)
def register_row_transform(kind, cls): _register("row_transform", kind, cls)


def mixer_class(spec): return _lookup("mixer", spec.kind)
def feed_forward_class(spec): return _lookup("feed_forward", spec.kind)
def norm_class(spec): return _lookup("norm", spec.kind)
def position_class(spec): return _lookup("position", spec.kind)
def block_class(kind: str): return _lookup("block", kind)
def row_transform_class(spec): return _lookup("row_transform", spec.kind)
