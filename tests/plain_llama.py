"""A plain, slow Llama decoder: whole sequences, no cache, one function for each part.

It is the answer key of the test-suite and shares no code with the engine: it reads a model
folder with its own few lines of safetensors parsing and computes everything with ordinary
torch tensor operations on the CPU, by default in float64.  Every function cites the lines
of the reference (paths relative to the reference's root) whose formula it states.
"""
from __future__ import annotations

import json
import math
import struct
from pathlib import Path

import torch

_ST_DTYPES = {"F32": torch.float32, "BF16": torch.bfloat16, "F16": torch.float16, "F64": torch.float64}


def read_model_folder(folder):
    """config.json as a dict and every tensor of model.safetensors by name.

    File format as the reference parses it (src/loader/safetensors.cpp:25-88): eight bytes of
    little-endian header length, a JSON header, offsets relative to the data region."""
    folder = Path(folder)
    cfg = json.loads((folder / "config.json").read_text())
    raw = (folder / "model.safetensors").read_bytes()
    (hlen,) = struct.unpack("<Q", raw[:8])
    header = json.loads(raw[8:8 + hlen])
    data = raw[8 + hlen:]
    tensors = {}
    for name, e in header.items():
        if name == "__metadata__":
            continue
        b, t = e["data_offsets"]
        flat = torch.frombuffer(bytearray(data[b:t]), dtype=_ST_DTYPES[e["dtype"]])
        tensors[name] = flat.reshape(e["shape"]).clone()
    return cfg, tensors


# --------------------------------------------------------------------------------------- parts
def rms_norm(x, weight, eps):
    """out = w * (x / sqrt(mean(x^2) + eps)); eps inside the root, the weight as it is (no 1 + w).
    Reference: src/kernels/kernels.cpp:72-83, tools/ref.py:26-28."""
    ms = (x * x).mean(dim=-1, keepdim=True)
    return weight * (x * torch.rsqrt(ms + eps))


def rope_inverse_frequencies(head_dim, theta, scaling=None):
    """f_k = theta^(-2k/head_dim) for k < head_dim/2, then the llama3 change per frequency.

    Written as the loop with three branches of src/kernels/kernels.cpp:142-158 (also
    tests/verify_kernels.py:305-317): wavelengths above original/low are divided by `factor`,
    those below original/high stay, the ones between are blended."""
    out = []
    for k in range(head_dim // 2):
        f = 1.0 / (float(theta) ** (2.0 * k / head_dim))
        if scaling is not None:
            factor = float(scaling["factor"])
            low = float(scaling["low_freq_factor"])
            high = float(scaling["high_freq_factor"])
            original = float(scaling["original_max_position_embeddings"])
            wavelength = 2.0 * math.pi / f
            if wavelength > original / low:
                f = f / factor
            elif not (wavelength < original / high):
                smooth = (original / wavelength - low) / (high - low)
                f = (1.0 - smooth) * f / factor + smooth * f
        out.append(f)
    return torch.tensor(out, dtype=torch.float64)


def rope_rotate(x, positions, inv_freq):
    """Rotation of the pairs (x[k], x[k + head_dim/2]) of every head by the angle pos * f_k:
    x[k] <- a*cos - b*sin, x[k + half] <- a*sin + b*cos.  x is [T, heads, head_dim].
    Reference: src/kernels/kernels.cpp:165-180 (HalfSplit), tools/ref.py:54-76."""
    half = x.shape[-1] // 2
    angle = positions.to(torch.float64)[:, None] * inv_freq[None, :]          # [T, half]
    cos = torch.cos(angle).to(x.dtype)[:, None, :]
    sin = torch.sin(angle).to(x.dtype)[:, None, :]
    a, b = x[..., :half], x[..., half:]
    return torch.cat([a * cos - b * sin, a * sin + b * cos], dim=-1)


def causal_attention(q, k, v, window=None):
    """Row i attends to rows j <= i of its own sequence (and j > i - window if a window is set);
    query head h uses key/value head h // (heads / kv_heads); scores are scaled by
    1/sqrt(head_dim) after the dot product; softmax over j; then the weighted sum of v.
    q is [T, heads, hd], k and v are [T, kv_heads, hd]; the result is [T, heads, hd].
    Reference: src/model/transformer.cpp:228-255, tools/ref.py:121-132."""
    T, n_heads, hd = q.shape
    group = n_heads // k.shape[1]
    out = torch.empty_like(q)
    rows = torch.arange(T)
    allowed = rows[None, :] <= rows[:, None]
    if window is not None:
        allowed &= rows[None, :] > rows[:, None] - window
    for h in range(n_heads):
        g = h // group
        scores = (q[:, h, :] @ k[:, g, :].T) * (1.0 / math.sqrt(hd))
        scores = scores.masked_fill(~allowed, float("-inf"))
        out[:, h, :] = torch.softmax(scores, dim=-1) @ v[:, g, :]
    return out


def swiglu(x, w_gate, w_up, w_down, store=lambda t: t):
    """down( silu(gate(x)) * up(x) ), silu(g) = g / (1 + exp(-g)).
    Reference: src/model/transformer.cpp:437-450, src/kernels/kernels.cpp:106-110."""
    g = x @ w_gate.T
    u = x @ w_up.T
    return store((g * (1.0 / (1.0 + torch.exp(-g)))) * u) @ w_down.T


# --------------------------------------------------------------------------------------- model
class PlainLlama:
    """The whole decoder over a whole sequence.  Order in a layer (src/model/transformer.cpp:385-450):
    x -> norm -> attention -> + x -> norm -> feed-forward -> + x; then the final norm and lm_head."""

    def __init__(self, folder, dtype=torch.float64, storage=None):
        """`storage=torch.bfloat16` rounds to bfloat16 wherever the engine's bfloat16 mode stores an
        activation as bfloat16 (inputs of the matrix products, rotated queries, cached keys and
        values, attention output, gated feed-forward output); sums, softmax, norms, rotation and
        the residual stream keep `dtype`.  With None nothing is rounded."""
        cfg, tensors = read_model_folder(folder)
        self.store = (lambda t: t.to(storage).to(dtype)) if storage is not None else (lambda t: t)
        self.cfg = cfg
        self.dtype = dtype
        self.w = {k: t.to(dtype) for k, t in tensors.items()}
        self.n_layers = cfg["num_hidden_layers"]
        self.n_heads = cfg["num_attention_heads"]
        self.n_kv = cfg.get("num_key_value_heads") or self.n_heads
        self.hd = cfg.get("head_dim") or cfg["hidden_size"] // self.n_heads
        self.eps = float(cfg.get("rms_norm_eps", 1e-6))            # src/loader/hf_checkpoint.cpp:128
        self.theta = float(cfg.get("rope_theta", 10000.0))         # src/loader/hf_checkpoint.cpp:127
        sc = cfg.get("rope_scaling")
        if sc and sc.get("rope_type", sc.get("type")) == "llama3":
            self.scaling = sc
        else:
            self.scaling = None
        self.tied = bool(cfg.get("tie_word_embeddings", False))    # src/loader/hf_checkpoint.cpp:133-134
        self.window = cfg.get("sliding_window")                    # not a Llama key; used by part tests only
        self.inv_freq = rope_inverse_frequencies(self.hd, self.theta, self.scaling)

    def hidden_states(self, tokens):
        w, T = self.w, len(tokens)
        pos = torch.arange(T)
        x = w["model.embed_tokens.weight"][torch.tensor(tokens)]
        for l in range(self.n_layers):
            p = f"model.layers.{l}."
            xb = self.store(rms_norm(x, w[p + "input_layernorm.weight"], self.eps))
            q = (xb @ w[p + "self_attn.q_proj.weight"].T).reshape(T, self.n_heads, self.hd)
            k = (xb @ w[p + "self_attn.k_proj.weight"].T).reshape(T, self.n_kv, self.hd)
            v = (xb @ w[p + "self_attn.v_proj.weight"].T).reshape(T, self.n_kv, self.hd)
            q = self.store(rope_rotate(q, pos, self.inv_freq))
            k = self.store(rope_rotate(k, pos, self.inv_freq))
            att = self.store(causal_attention(q, k, self.store(v), self.window)).reshape(T, self.n_heads * self.hd)
            x = x + att @ w[p + "self_attn.o_proj.weight"].T
            xb = self.store(rms_norm(x, w[p + "post_attention_layernorm.weight"], self.eps))
            x = x + swiglu(xb, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                           w[p + "mlp.down_proj.weight"], self.store)
        return x

    def logits(self, tokens):
        """Logits [T, vocab] at every position of one sequence (src/model/transformer.cpp:453-474)."""
        x = self.store(rms_norm(self.hidden_states(tokens), self.w["model.norm.weight"], self.eps))
        head = self.w["model.embed_tokens.weight"] if self.tied else self.w["lm_head.weight"]
        return x @ head.T

    def logits_at(self, tokens, positions):
        """The rows `positions` of `logits(tokens)`, with the head applied to those rows only."""
        x = self.store(rms_norm(self.hidden_states(tokens)[torch.tensor(list(positions))], self.w["model.norm.weight"], self.eps))
        head = self.w["model.embed_tokens.weight"] if self.tied else self.w["lm_head.weight"]
        return x @ head.T

    def with_storage(self, storage):
        """The same model (the weights are shared, not read again) rounding to `storage` where the engine stores it."""
        other = PlainLlama.__new__(PlainLlama)
        other.__dict__.update(self.__dict__)
        other.store = (lambda t: t.to(storage).to(self.dtype)) if storage is not None else (lambda t: t)
        return other

    def greedy(self, prompt, n_new):
        """Greedy continuation, recomputing the whole sequence for every new token."""
        toks = list(prompt)
        for _ in range(n_new):
            toks.append(int(torch.argmax(self.logits(toks)[-1])))
        return toks[len(prompt):]


def scaled_error(got, want):
    """max|got - want| / max(1, max|want|): the measure of tests/verify_forward.py:72-77."""
    got = torch.as_tensor(got, dtype=torch.float64)
    want = torch.as_tensor(want, dtype=torch.float64)
    return float((got - want).abs().max() / max(1.0, float(want.abs().max())))
