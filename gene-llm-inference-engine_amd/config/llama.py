"""Typed configuration of the Llama dense decoder, read from its own config.json keys.

Keys, defaults and refusals follow the reference's parser (src/loader/hf_checkpoint.cpp:28-136):
required hidden_size, intermediate_size, num_hidden_layers, num_attention_heads, vocab_size;
optional num_key_value_heads (= heads), max_position_embeddings (2048), head_dim
(hidden / heads), rope_theta (10000), rms_norm_eps (1e-6), rope_scaling (none),
tie_word_embeddings (false).
"""
from __future__ import annotations

import json
import math
from dataclasses import dataclass, asdict
from typing import Optional

from .errors import ConfigError
from .registry import register_architecture
from .spec import AttentionSpec, LayerSpec, ModelSpec, RmsNormSpec, RotarySpec, RunEntry, SwiGluSpec


_MAX_INT = 100_000_000   # src/loader/hf_checkpoint.cpp:31


def _is_int(v):
    return isinstance(v, int) and not isinstance(v, bool) or (isinstance(v, float) and v == int(v))


def _required_int(cfg, key):
    if key not in cfg:
        raise ConfigError(f"config.json has no '{key}'")
    return _checked_int(cfg[key], key)


def _checked_int(v, key):
    if not _is_int(v) or not 0 < int(v) <= _MAX_INT:
        raise ConfigError(f"config.json: '{key}' has an invalid value")
    return int(v)


def _optional_int(cfg, key, fallback):
    v = cfg.get(key)
    return fallback if v is None else _checked_int(v, key)


def _optional_number(cfg, key, fallback):
    v = cfg.get(key)
    if v is None:
        return fallback
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(f"config.json: '{key}' is not a number")
    return float(v)


@dataclass(frozen=True)
class Llama3Scaling:
    """Per-frequency stretch of rotary frequencies (reference: src/common/rope_style.h:13-19)."""
    factor: float
    low_freq_factor: float
    high_freq_factor: float
    original_max_position_embeddings: int


def rotary_frequencies(head_dim: int, theta: float, scaling: Optional[Llama3Scaling] = None):
    """f_k = theta^(-2k/head_dim) in 64-bit, and with scaling the reference's rule per frequency
    (src/kernels/kernels.cpp:142-158): a wavelength 2*pi/f above original/low_freq_factor divides f by `factor`, one
    below original/high_freq_factor leaves it, and between the two f is blended."""
    out = []
    for k in range(head_dim // 2):
        f = 1.0 / math.pow(float(theta), 2.0 * k / head_dim)
        if scaling is not None:
            wavelength = 6.283185307179586476925 / f
            original = float(scaling.original_max_position_embeddings)
            if wavelength > original / scaling.low_freq_factor:
                f /= scaling.factor
            elif not wavelength < original / scaling.high_freq_factor:
                smooth = (original / wavelength - scaling.low_freq_factor) / (scaling.high_freq_factor - scaling.low_freq_factor)
                f = (1.0 - smooth) * f / scaling.factor + smooth * f
        out.append(f)
    return tuple(out)


def _parse_rope_scaling(s) -> Optional[Llama3Scaling]:
    """null, absent and type "default" mean none; "llama3" needs all four numbers; every other
    type is refused (src/loader/hf_checkpoint.cpp:55-90)."""
    if s is None:
        return None
    if not isinstance(s, dict):
        raise ConfigError("rope_scaling is not an object")
    kind = None
    for key in ("rope_type", "type"):
        if key in s:
            if not isinstance(s[key], str):
                raise ConfigError(f"rope_scaling.{key} is not a string")
            kind = s[key]
            break
    if kind == "default":
        return None
    if kind != "llama3":
        raise ConfigError(f"rope_scaling type '{kind if kind is not None else ''}' is not supported (only 'llama3')")

    def number(key):
        v = s.get(key)
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"rope_scaling.{key} is required for type 'llama3'")
        return float(v)

    factor, low, high = number("factor"), number("low_freq_factor"), number("high_freq_factor")
    original = number("original_max_position_embeddings")
    if not factor >= 1.0:
        raise ConfigError("rope_scaling.factor must be >= 1")
    if not low > 0.0 or not high > low:
        raise ConfigError("rope_scaling needs 0 < low_freq_factor < high_freq_factor")
    if not original >= 1.0 or original > 1e9 or original != int(original):
        raise ConfigError("rope_scaling.original_max_position_embeddings must be a positive integer")
    return Llama3Scaling(factor, low, high, int(original))


@dataclass(frozen=True)
class LlamaConfig:
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    vocab_size: int
    max_position_embeddings: int
    rope_theta: float
    rms_norm_eps: float
    rope_scaling: Optional[Llama3Scaling]
    tie_word_embeddings: bool

    architecture = "LlamaForCausalLM"
    model_type = "llama"

    @classmethod
    def from_dict(cls, cfg: dict) -> "LlamaConfig":
        if not isinstance(cfg, dict):
            raise ConfigError("config.json is not a JSON object")
        mt = cfg.get("model_type")
        if isinstance(mt, str) and mt != cls.model_type:
            raise ConfigError(f"unsupported model_type '{mt}' for {cls.architecture} (expected '{cls.model_type}')")
        act = cfg.get("hidden_act")
        if isinstance(act, str) and act != "silu":
            raise ConfigError(f"unsupported hidden_act '{act}'")
        for bias in ("attention_bias", "mlp_bias"):
            if cfg.get(bias) is True:
                raise ConfigError(f"{bias} = true is not supported")

        hidden = _required_int(cfg, "hidden_size")
        inter = _required_int(cfg, "intermediate_size")
        layers = _required_int(cfg, "num_hidden_layers")
        heads = _required_int(cfg, "num_attention_heads")
        kv_heads = _optional_int(cfg, "num_key_value_heads", heads)
        vocab = _required_int(cfg, "vocab_size")
        max_pos = _optional_int(cfg, "max_position_embeddings", 2048)
        head_dim = _optional_int(cfg, "head_dim", 0)
        if head_dim == 0:
            if hidden % heads != 0:
                raise ConfigError("hidden_size is not divisible by num_attention_heads")
            head_dim = hidden // heads
        if heads % kv_heads != 0:
            raise ConfigError("num_attention_heads must be divisible by num_key_value_heads")
        if head_dim % 2 != 0:
            raise ConfigError("head_dim must be even (RoPE rotates pairs)")
        tie = cfg.get("tie_word_embeddings")
        return cls(
            hidden_size=hidden, intermediate_size=inter, num_hidden_layers=layers,
            num_attention_heads=heads, num_key_value_heads=kv_heads, head_dim=head_dim,
            vocab_size=vocab, max_position_embeddings=max_pos,
            rope_theta=_optional_number(cfg, "rope_theta", 10000.0),
            rms_norm_eps=_optional_number(cfg, "rms_norm_eps", 1e-6),
            rope_scaling=_parse_rope_scaling(cfg.get("rope_scaling")),
            tie_word_embeddings=tie is True,
        )

    def to_dict(self) -> dict:
        """config.json content that `from_dict` reads back to an equal configuration."""
        d = asdict(self)
        d["rope_scaling"] = None if self.rope_scaling is None else {"rope_type": "llama3", **asdict(self.rope_scaling)}
        return {"architectures": [self.architecture], "model_type": self.model_type, "hidden_act": "silu",
                "attention_bias": False, "mlp_bias": False, **d}

    def to_json(self) -> str:
        return json.dumps(self.to_dict(), indent=2)

    # derived sizes (reference: src/loader/checkpoint.h:93-96)
    @property
    def attn_dim(self):
        return self.num_attention_heads * self.head_dim

    @property
    def kv_dim(self):
        return self.num_key_value_heads * self.head_dim

    def model_spec(self) -> ModelSpec:
        """The decoder as parts: per layer pre-norm attention with rotary positions and a SwiGLU
        feed-forward, tensor names as a Hugging Face Llama folder stores them
        (src/loader/hf_checkpoint.cpp:214-235)."""
        rotary = RotarySpec(self.head_dim, self.rope_theta,
                            None if self.rope_scaling is None else rotary_frequencies(self.head_dim, self.rope_theta, self.rope_scaling))
        layers = []
        for l in range(self.num_hidden_layers):
            p = f"model.layers.{l}."
            layers.append(LayerSpec(
                mixer=AttentionSpec(
                    hidden_size=self.hidden_size, n_heads=self.num_attention_heads,
                    n_kv_heads=self.num_key_value_heads, head_dim=self.head_dim,
                    q_proj=p + "self_attn.q_proj.weight", k_proj=p + "self_attn.k_proj.weight",
                    v_proj=p + "self_attn.v_proj.weight", o_proj=p + "self_attn.o_proj.weight",
                    position=rotary, window=None),
                feed_forward=SwiGluSpec(
                    hidden_size=self.hidden_size, intermediate_size=self.intermediate_size,
                    gate_proj=p + "mlp.gate_proj.weight", up_proj=p + "mlp.up_proj.weight",
                    down_proj=p + "mlp.down_proj.weight"),
                mixer_norm=RmsNormSpec(self.hidden_size, self.rms_norm_eps, p + "input_layernorm.weight"),
                feed_forward_norm=RmsNormSpec(self.hidden_size, self.rms_norm_eps, p + "post_attention_layernorm.weight"),
                block="prenorm"))
        embedding = "model.embed_tokens.weight"
        ignorable = [r".*\.rotary_emb\.inv_freq"]
        if self.tie_word_embeddings:
            ignorable.append(r"lm_head\.weight")       # a tied file may still carry one; it is not used
        return ModelSpec(
            architecture=self.architecture, vocab_size=self.vocab_size, hidden_size=self.hidden_size,
            max_positions=self.max_position_embeddings, embedding=embedding,
            final_norm=RmsNormSpec(self.hidden_size, self.rms_norm_eps, "model.norm.weight"),
            lm_head=embedding if self.tie_word_embeddings else "lm_head.weight",
            layers=tuple(layers), run_order=tuple(RunEntry(l) for l in range(self.num_hidden_layers)),
            ignorable_tensors=tuple(ignorable))


register_architecture(LlamaConfig.architecture, LlamaConfig, model_type=LlamaConfig.model_type)
