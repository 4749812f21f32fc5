"""Architecture-neutral description of a model: what the engine builds from.

An architecture's own configuration class (for instance `LlamaConfig`) reads config.json and
translates itself into a `ModelSpec`: a list of layers, each naming its mixer, feed-forward,
norms and position encoding with all sizes, constants and tensor names as fields, and a run
order.  Nothing below this file knows which architecture a spec came from.

Every part spec is a frozen dataclass with a class attribute `kind`; the parts registry maps
`kind` to the class that implements it, so a new kind of part needs a spec class, an
implementation and one `register_*` call.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, ClassVar, Optional, Tuple


@dataclass(frozen=True)
class RotarySpec:
    """Rotation of the pairs (k, k + head_dim/2) of every head by pos * f_k, with f_k = theta^(-2k/head_dim) unless the
    architecture gives its own `frequencies` (head_dim/2 numbers: whatever rule stretches or blends them is the
    architecture's, applied where it builds this spec)."""
    kind: ClassVar[str] = "rotary_half_split"
    head_dim: int
    theta: float
    frequencies: Optional[Tuple[float, ...]] = None

    def __post_init__(self):
        if self.frequencies is not None and len(self.frequencies) != self.head_dim // 2:
            raise ValueError(f"a rotation of heads of {self.head_dim} channels needs {self.head_dim // 2} frequencies, not {len(self.frequencies)}")


@dataclass(frozen=True)
class RmsNormSpec:
    kind: ClassVar[str] = "rmsnorm"
    size: int
    eps: float
    weight: str                      # tensor name


@dataclass(frozen=True)
class AttentionSpec:
    """Causal attention with grouped key/value heads over a paged cache."""
    kind: ClassVar[str] = "attention"
    hidden_size: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    q_proj: str
    k_proj: str
    v_proj: str
    o_proj: str
    position: Optional[Any] = None   # a position-encoding spec, or None for no rotation
    window: Optional[int] = None     # keys further back than this many positions are not seen


@dataclass(frozen=True)
class SwiGluSpec:
    """down( silu(gate(x)) * up(x) ), no biases."""
    kind: ClassVar[str] = "swiglu"
    hidden_size: int
    intermediate_size: int
    gate_proj: str
    up_proj: str
    down_proj: str


@dataclass(frozen=True)
class ScaleSpec:
    """Rows multiplied by a constant (for instance a token table that is stored unscaled)."""
    kind: ClassVar[str] = "scale"
    factor: float


@dataclass(frozen=True)
class SoftCapSpec:
    """x <- cap * tanh(x / cap): values kept within (-cap, cap)."""
    kind: ClassVar[str] = "softcap"
    cap: float


@dataclass(frozen=True)
class LayerSpec:
    """One layer: which parts, and in which arrangement (`block`) they are wired."""
    mixer: Any
    feed_forward: Any
    mixer_norm: Any
    feed_forward_norm: Any
    block: str = "prenorm"


@dataclass(frozen=True)
class RunEntry:
    """One position of the run order.  `layer` indexes `ModelSpec.layers` (a layer may be named by
    several entries).  `cache_of` is None when the entry keeps a cache of its own, or the index of
    an earlier entry whose cache it reads without writing."""
    layer: int
    cache_of: Optional[int] = None


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden_size: int
    max_positions: int
    embedding: str                       # tensor name of the token table [vocab, hidden]
    final_norm: Any
    lm_head: str                         # tensor name; the embedding's name when tied
    layers: Tuple[LayerSpec, ...]
    run_order: Tuple[RunEntry, ...]
    ignorable_tensors: Tuple[str, ...] = field(default=())   # regular expressions of names a file may hold unused
    after_embedding: Tuple[Any, ...] = field(default=())     # row-transform specs applied, in order, to the rows of the token table
    after_head: Tuple[Any, ...] = field(default=())          # ... and to the logits

    def __post_init__(self):
        for i, e in enumerate(self.run_order):
            if not 0 <= e.layer < len(self.layers):
                raise ValueError(f"run order entry {i} names layer {e.layer}, but there are {len(self.layers)} layers")
            if e.cache_of is not None:
                if not 0 <= e.cache_of < i:
                    raise ValueError(f"run order entry {i} reads the cache of entry {e.cache_of}, which does not run before it")
                if self.run_order[e.cache_of].cache_of is not None:
                    raise ValueError(f"run order entry {i} reads the cache of entry {e.cache_of}, which has none of its own")
