"""A toy architecture that exists only in the tests, to show that parts, layer order and cache
needs are data: it is registered, built, loaded and stepped through the framework's public
interfaces without a change to the framework's files.

Layers (pre-norm blocks with RMS norms unless said otherwise): 0 full attention whose positions are encoded by a
rule and a pairing of its own (neighbouring channels (2i, 2i+1) of the first `rotary_dim` channels of a head are
turned by pos * step * (i + 1), the rest of the head is left alone: the encoding applies itself to q and k),
1 windowed attention with half-split pairs but angles of its own (pos * step * (k + 1): the encoding hands the
attention kernels its cosines and sines), 2 a "decay" mixer
with a state of its own (s <- decay * s + h per row, out = W s), each followed by SwiGLU, layer 2
in a block arrangement of its own (mixer and feed-forward both read one norm of the block's input, a
norm that also removes the mean, and both add onto the residual stream); 3 a
second decay mixer followed by a feed-forward with routing (a router picks one of three small
SwiGLU experts per row and scales it by the router's probability of it).  Run order: 3, 0, 1, 2,
then layer 0 once more (a cache of its own) and layer 1 once more reading the pages of its first
run.  Layer 3 runs first so that the router sees values computed in 32-bit on both sides of the
comparison (embedding, norm, decay mixer): in bfloat16 the engine and the plain model then take
the same expert unless two router logits agree to six digits.  The rows of the token table are scaled by a
constant before the first layer and the logits are capped softly (the model's two row-transform places).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import ClassVar

import torch

from geneinfer_amd.cache import StateNeed
from geneinfer_amd.config import (AttentionSpec, LayerSpec, ModelSpec, RmsNormSpec, RunEntry, ScaleSpec, SoftCapSpec, SwiGluSpec,
                                  register_architecture)
from geneinfer_amd.parts import (FeedForward, Mixer, Norm, PositionEncoding, feed_forward_class, mixer_class, norm_class, register_block,
                                 register_feed_forward, register_mixer, register_norm, register_position_encoding)
from geneinfer_amd.weights import TensorNeed
from plain_llama import causal_attention, rms_norm, rope_rotate, swiglu


@dataclass(frozen=True)
class DecaySpec:
    kind: ClassVar[str] = "toy_decay"
    hidden_size: int
    decay: float
    weight: str


class DecayMixer(Mixer):
    """State per request: s [hidden] in 32-bit.  Rows of a request are taken in order; the state is
    read at the start of the request's rows and written back after them.

    Which slot a request's state lies in is read on the device (the slot of the request's first row), and only the
    cut of the step into requests (where each begins, how many rows it has) comes from the host's lists: that cut is
    part of a captured pass's shape, the slots are not, so the mixer may be captured and replayed."""
    graph_safe = True

    def __init__(self, spec, tensors, dtype, device):
        super().__init__(spec, tensors, dtype, device)
        self.w = tensors[spec.weight].float()
        self.in_dtype = torch.float32

    @classmethod
    def tensor_needs(cls, spec):
        return [TensorNeed(spec.weight, (spec.hidden_size, spec.hidden_size))]

    @classmethod
    def cache_need(cls, spec):
        return StateNeed((spec.hidden_size,), torch.float32)

    def forward(self, h, residual, ctx, cache):
        for start, n in zip(ctx.seg_start, ctx.seg_len):
            slot = ctx.row_slot[start:start + 1].long()
            s = cache.state.index_select(0, slot)[0]
            for i in range(start, start + n):
                s = self.spec.decay * s + h[i].float()
                residual[i] += self.w @ s
            cache.state.index_copy_(0, slot, s[None])


@dataclass(frozen=True)
class CenteredNormSpec:
    kind: ClassVar[str] = "toy_centered_norm"
    size: int
    eps: float
    weight: str


class CenteredNorm(Norm):
    """w * (x - mean(x)) / sqrt(var(x) + eps), in 32-bit; the result is stored as the consumer asks."""
    graph_safe = True

    def __init__(self, spec, tensors, dtype, device):
        super().__init__(spec, tensors, dtype, device)
        self.weight = tensors[spec.weight].float()

    @classmethod
    def tensor_needs(cls, spec):
        return [TensorNeed(spec.weight, (spec.size,), "norm")]

    def __call__(self, x, out_dtype, rows=None):
        x = x if rows is None else x[rows.long()]
        centered = x - x.mean(dim=-1, keepdim=True)
        return (self.weight * centered * torch.rsqrt(centered.square().mean(dim=-1, keepdim=True) + self.spec.eps)).to(out_dtype)


class ParallelBlock:
    """x += mixer(norm(x)) + feed_forward(norm(x)): one norm, read by both halves.  What the model asks of a block:
    `tensor_needs(layer_spec)`, `cache_need(layer_spec)`, `forward(x, ctx, cache)`, `graph_safe`."""

    @property
    def graph_safe(self):
        return all(getattr(p, "graph_safe", False) for p in (self.mixer_norm, self.mixer, self.feed_forward))

    def __init__(self, spec, tensors, dtype, device):
        self.spec = spec
        self.mixer_norm = norm_class(spec.mixer_norm)(spec.mixer_norm, tensors, dtype, device)
        self.mixer = mixer_class(spec.mixer)(spec.mixer, tensors, dtype, device)
        self.feed_forward = feed_forward_class(spec.feed_forward)(spec.feed_forward, tensors, dtype, device)

    @classmethod
    def tensor_needs(cls, spec):
        return (norm_class(spec.mixer_norm).tensor_needs(spec.mixer_norm) + mixer_class(spec.mixer).tensor_needs(spec.mixer) +
                feed_forward_class(spec.feed_forward).tensor_needs(spec.feed_forward))

    @classmethod
    def cache_need(cls, spec):
        return mixer_class(spec.mixer).cache_need(spec.mixer)

    def forward(self, x, ctx, cache):
        for_mixer = self.mixer_norm(x, getattr(self.mixer, "in_dtype", ctx.dtype))
        for_feed_forward = self.mixer_norm(x, getattr(self.feed_forward, "in_dtype", ctx.dtype))       # before the mixer changes x
        self.mixer.forward(for_mixer, x, ctx, cache)
        self.feed_forward.forward(for_feed_forward, x, ctx)


@dataclass(frozen=True)
class LinearAnglesSpec:
    kind: ClassVar[str] = "toy_linear_angles"
    head_dim: int
    step: float


class LinearAngles(PositionEncoding):
    """Pair (k, k + head_dim/2) of a head is turned by pos * step * (k + 1): a rotation of half-split pairs over the
    whole head, so the attention kernels apply it themselves from `half_split_tables(ctx) -> (cos, sin)`, float32
    [rows, head_dim / 2]."""
    graph_safe = True                                         # everything step-dependent is read on the device

    def half_split_tables(self, ctx):
        key = ("toy_linear_angles", self.spec)
        if key not in ctx.memo:
            k = torch.arange(1, self.spec.head_dim // 2 + 1, dtype=torch.float64, device=ctx.device)
            angles = ctx.row_pos.double()[:, None] * (self.spec.step * k)[None, :]
            ctx.memo[key] = (torch.cos(angles).float().contiguous(), torch.sin(angles).float().contiguous())
        return ctx.memo[key]


@dataclass(frozen=True)
class NeighbourPairsSpec:
    kind: ClassVar[str] = "toy_neighbour_pairs"
    head_dim: int
    rotary_dim: int                   # the first so many channels of a head are turned, in pairs (2i, 2i + 1)
    step: float


class NeighbourPairs(PositionEncoding):
    """Another pairing, and only a part of the head: no half-split tables, so the attention part calls `apply` with
    the rows' float32 queries and keys (column ranges of the stacked product) and stores them as they come back."""
    graph_safe = True

    def apply(self, q, k, ctx, n_heads, n_kv_heads, head_dim):
        assert head_dim == self.spec.head_dim and q.dtype == torch.float32 and q.shape == (ctx.n_rows, n_heads * head_dim)
        half = self.spec.rotary_dim // 2
        i = torch.arange(1, half + 1, dtype=torch.float64, device=ctx.device)
        angles = ctx.row_pos.double()[:, None] * (self.spec.step * i)[None, :]
        cos, sin = torch.cos(angles).float()[:, None, :], torch.sin(angles).float()[:, None, :]
        for x, heads in ((q, n_heads), (k, n_kv_heads)):
            if x is None:
                continue
            v = x.unflatten(1, (heads, head_dim))                 # a view: x may be a column range of a wider tensor
            a, b = v[..., 0:2 * half:2].clone(), v[..., 1:2 * half:2].clone()
            v[..., 0:2 * half:2] = a * cos - b * sin
            v[..., 1:2 * half:2] = a * sin + b * cos


def turn_neighbour_pairs(x, positions, rotary_dim, step):
    """The plain statement of NeighbourPairs for a whole sequence; x is [T, heads, head_dim]."""
    half = rotary_dim // 2
    angles = positions.double()[:, None] * (step * torch.arange(1, half + 1, dtype=torch.float64))[None, :]
    cos, sin = torch.cos(angles).to(x.dtype)[:, None, :], torch.sin(angles).to(x.dtype)[:, None, :]
    out = x.clone()
    a, b = x[..., 0:2 * half:2], x[..., 1:2 * half:2]
    out[..., 0:2 * half:2] = a * cos - b * sin
    out[..., 1:2 * half:2] = a * sin + b * cos
    return out


@dataclass(frozen=True)
class RoutedSpec:
    kind: ClassVar[str] = "toy_routed"
    hidden_size: int
    intermediate_size: int
    n_experts: int
    prefix: str                       # tensors: prefix + "router", prefix + "e{i}.gate" / ".up" / ".down"


class RoutedFeedForward(FeedForward):
    """Per row: the expert with the largest router logit (the lowest index among equals), scaled by its softmax
    probability.  Everything in 32-bit.  Every expert is worked out for every row and the chosen one's result kept, so
    that no shape depends on the routing and the pass can be captured; `gathered=True` takes each expert's rows out
    instead (what a real one would do; its shapes follow the data, so such a part says graph_safe = False)."""
    gathered = False

    @property
    def graph_safe(self):
        return not self.gathered

    def __init__(self, spec, tensors, dtype, device):
        super().__init__(spec, tensors, dtype, device)
        self.router = tensors[spec.prefix + "router"].float()
        self.experts = [tuple(tensors[f"{spec.prefix}e{i}.{n}"].float() for n in ("gate", "up", "down")) for i in range(spec.n_experts)]
        self.in_dtype = torch.float32

    @classmethod
    def tensor_needs(cls, spec):
        d, inter = spec.hidden_size, spec.intermediate_size
        needs = [TensorNeed(spec.prefix + "router", (spec.n_experts, d))]
        for i in range(spec.n_experts):
            needs += [TensorNeed(f"{spec.prefix}e{i}.gate", (inter, d)), TensorNeed(f"{spec.prefix}e{i}.up", (inter, d)),
                      TensorNeed(f"{spec.prefix}e{i}.down", (d, inter))]
        return needs

    def forward(self, h, residual, ctx):
        h = h.float()
        logits = h @ self.router.T
        chosen = torch.argmax(logits, dim=-1)                 # the first of equal maxima
        share = torch.softmax(logits, dim=-1).gather(1, chosen[:, None])
        for i, (gate, up, down) in enumerate(self.experts):
            if self.gathered:
                rows = torch.nonzero(chosen == i).flatten()
                if rows.numel():
                    x = h[rows]
                    residual[rows] += share[rows] * ((torch.nn.functional.silu(x @ gate.T) * (x @ up.T)) @ down.T)
            else:
                result = (torch.nn.functional.silu(h @ gate.T) * (h @ up.T)) @ down.T
                residual += torch.where((chosen == i)[:, None], share * result, torch.zeros_like(result))


@dataclass(frozen=True)
class ToyConfig:
    hidden_size: int = 48
    intermediate_size: int = 80
    num_attention_heads: int = 3
    num_key_value_heads: int = 1
    head_dim: int = 16
    vocab_size: int = 200
    window: int = 6
    decay: float = 0.7
    angle_step: float = 0.05
    rotary_dim: int = 12
    embedding_scale: float = 1.5
    logit_cap: float = 3.0
    num_experts: int = 3
    expert_intermediate_size: int = 24
    rms_norm_eps: float = 1e-5
    max_position_embeddings: int = 256

    architecture = "ToyMixedForCausalLM"

    @classmethod
    def from_dict(cls, d):
        return cls(**{k: d[k] for k in cls.__dataclass_fields__ if k in d})

    def to_dict(self):
        return {"architectures": [self.architecture], "model_type": "toy_mixed", **{k: getattr(self, k) for k in self.__dataclass_fields__}}

    def model_spec(self) -> ModelSpec:
        d = self.hidden_size
        def attention(l, window, position):
            p = f"layers.{l}.attn."
            return AttentionSpec(d, self.num_attention_heads, self.num_key_value_heads, self.head_dim, p + "q", p + "k", p + "v", p + "o",
                                 position=position, window=window)
        def rest(l, mixer, feed_forward=None, parallel=False):
            p = f"layers.{l}."
            feed_forward = feed_forward or SwiGluSpec(d, self.intermediate_size, p + "ff.gate", p + "ff.up", p + "ff.down")
            if parallel:
                norm = CenteredNormSpec(d, self.rms_norm_eps, p + "norm1")
                return LayerSpec(mixer=mixer, feed_forward=feed_forward, mixer_norm=norm, feed_forward_norm=norm, block="toy_parallel")
            return LayerSpec(mixer=mixer, feed_forward=feed_forward,
                             mixer_norm=RmsNormSpec(d, self.rms_norm_eps, p + "norm1"), feed_forward_norm=RmsNormSpec(d, self.rms_norm_eps, p + "norm2"))
        layers = (rest(0, attention(0, None, NeighbourPairsSpec(self.head_dim, self.rotary_dim, self.angle_step))),
                  rest(1, attention(1, self.window, LinearAnglesSpec(self.head_dim, self.angle_step))),
                  rest(2, DecaySpec(d, self.decay, "layers.2.decay.w"), parallel=True),
                  rest(3, DecaySpec(d, self.decay, "layers.3.decay.w"), RoutedSpec(d, self.expert_intermediate_size, self.num_experts, "layers.3.moe.")))
        order = (RunEntry(3), RunEntry(0), RunEntry(1), RunEntry(2), RunEntry(0), RunEntry(1, cache_of=2))
        return ModelSpec(architecture=self.architecture, vocab_size=self.vocab_size, hidden_size=d, max_positions=self.max_position_embeddings,
                         embedding="embed", final_norm=RmsNormSpec(d, self.rms_norm_eps, "final_norm"), lm_head="head", layers=layers,
                         run_order=order, after_embedding=(ScaleSpec(self.embedding_scale),), after_head=(SoftCapSpec(self.logit_cap),))


def register():
    """Idempotent: the registries refuse a second class under a name, not the same class again."""
    register_mixer("toy_decay", DecayMixer)
    register_feed_forward("toy_routed", RoutedFeedForward)
    register_position_encoding("toy_linear_angles", LinearAngles)
    register_position_encoding("toy_neighbour_pairs", NeighbourPairs)
    register_norm("toy_centered_norm", CenteredNorm)
    register_block("toy_parallel", ParallelBlock)
    register_architecture(ToyConfig.architecture, ToyConfig, model_type="toy_mixed")


def router_logits(cfg: ToyConfig, w: dict, tokens, dtype=torch.float64):
    """What the router of layer 3 (the first to run) sees for a whole sequence, from the plain parts."""
    w = {k: v.to(dtype) for k, v in w.items()}
    x = w["embed"][torch.tensor(tokens)] * cfg.embedding_scale
    xb = rms_norm(x, w["layers.3.norm1"], cfg.rms_norm_eps)
    s, outs = torch.zeros(cfg.hidden_size, dtype=dtype), []
    for t in range(len(tokens)):
        s = cfg.decay * s + xb[t]
        outs.append(w["layers.3.decay.w"] @ s)
    x = x + torch.stack(outs)
    return rms_norm(x, w["layers.3.norm2"], cfg.rms_norm_eps) @ w["layers.3.moe.router"].T


def plain_logits(cfg: ToyConfig, w: dict, tokens, dtype=torch.float64, store=lambda t: t):
    """The toy model over a whole sequence with the plain parts (no cache, no state slots)."""
    w = {k: v.to(dtype) for k, v in w.items()}
    T, H, KV, hd = len(tokens), cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    pos = torch.arange(T)
    linear_angles = cfg.angle_step * torch.arange(1, hd // 2 + 1, dtype=torch.float64)
    turn = {0: lambda v: turn_neighbour_pairs(v, pos, cfg.rotary_dim, cfg.angle_step), 1: lambda v: rope_rotate(v, pos, linear_angles)}
    x = w["embed"][torch.tensor(tokens)] * cfg.embedding_scale
    spec = cfg.model_spec()
    kept = {}
    for i, entry in enumerate(spec.run_order):
        l, p = entry.layer, f"layers.{entry.layer}."
        if l == 2:                                            # the parallel block: one centered norm feeds both halves
            c = x - x.mean(dim=-1, keepdim=True)
            xb = w[p + "norm1"] * c * torch.rsqrt(c.square().mean(dim=-1, keepdim=True) + cfg.rms_norm_eps)
            s, outs = torch.zeros(cfg.hidden_size, dtype=dtype), []
            for t in range(T):
                s = cfg.decay * s + xb[t]
                outs.append(w[p + "decay.w"] @ s)
            x = x + torch.stack(outs) + swiglu(store(xb), w[p + "ff.gate"], w[p + "ff.up"], w[p + "ff.down"], store)
            continue
        xb = rms_norm(x, w[p + "norm1"], cfg.rms_norm_eps)
        if l >= 2:
            s, outs = torch.zeros(cfg.hidden_size, dtype=dtype), []
            for t in range(T):
                s = cfg.decay * s + xb[t]
                outs.append(w[p + "decay.w"] @ s)
            x = x + torch.stack(outs)
        else:
            xb = store(xb)
            q = store(turn[l]((xb @ w[p + "attn.q"].T).reshape(T, H, hd)))
            if entry.cache_of is None:
                k = store(turn[l]((xb @ w[p + "attn.k"].T).reshape(T, KV, hd)))
                v = store((xb @ w[p + "attn.v"].T).reshape(T, KV, hd))
                kept[i] = (k, v)
            else:
                k, v = kept[entry.cache_of]
            att = store(causal_attention(q, k, v, cfg.window if l == 1 else None)).reshape(T, H * hd)
            x = x + att @ w[p + "attn.o"].T
        if l == 3:                                            # the routed feed-forward: one expert per row, in 32-bit on the device
            xb = rms_norm(x, w[p + "norm2"], cfg.rms_norm_eps)
            logits = xb @ w[p + "moe.router"].T
            for t in range(T):
                e = int(torch.argmax(logits[t]))
                share = torch.softmax(logits[t], dim=-1)[e]
                x[t] = x[t] + share * swiglu(xb[t:t + 1], w[f"{p}moe.e{e}.gate"], w[f"{p}moe.e{e}.up"], w[f"{p}moe.e{e}.down"], lambda v: v)[0]
            continue
        xb = store(rms_norm(x, w[p + "norm2"], cfg.rms_norm_eps))
        x = x + swiglu(xb, w[p + "ff.gate"], w[p + "ff.up"], w[p + "ff.down"], store)
    logits = store(rms_norm(x, w["final_norm"], cfg.rms_norm_eps)) @ w["head"].T
    return cfg.logit_cap * torch.tanh(logits / cfg.logit_cap)
