"""Tiny model folders for the tests, written without any of the engine's code: config.json and a
safetensors file made by hand here, so that the engine's loader reads a file it did not write.

Weights are drawn as the reference's test generator draws them (tools/make_dummy_hf.py:99-106):
matrices 0.2 * N(0, 1) (large enough that logits are of order one and relative errors mean
something), norm weights 1 + 0.1 * N(0, 1), stored in a shuffled order."""
from __future__ import annotations

import json
import struct
from pathlib import Path

import numpy as np
import torch

# Two configurations that differ in every size and option, and a third with odd sizes.
TINY_A = dict(hidden_size=64, intermediate_size=192, num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2,
              vocab_size=256, rope_theta=10000.0, rope_scaling=None, rms_norm_eps=1e-5, tie_word_embeddings=True,
              max_position_embeddings=512)
TINY_B = dict(hidden_size=96, intermediate_size=160, num_hidden_layers=3, num_attention_heads=3, num_key_value_heads=1,
              head_dim=32, vocab_size=384, rope_theta=500000.0,
              rope_scaling=dict(rope_type="llama3", factor=4.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                original_max_position_embeddings=32),
              rms_norm_eps=1e-6, tie_word_embeddings=False, max_position_embeddings=1024)
TINY_C = dict(hidden_size=80, intermediate_size=112, num_hidden_layers=1, num_attention_heads=6, num_key_value_heads=3,
              head_dim=48, vocab_size=301, rope_theta=25000.0, rope_scaling=None, rms_norm_eps=3e-5,
              tie_word_embeddings=False, max_position_embeddings=256)
# A fourth whose head size and page size the matrix-core attention kernels take (A, B and C run the exact attention
# kernels in both dtypes: pages of 4 and 8 positions, heads of 48 channels), with prompts long enough for several tiles.
TINY_D = dict(hidden_size=128, intermediate_size=208, num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=2,
              head_dim=64, vocab_size=515, rope_theta=1000000.0, rope_scaling=None, rms_norm_eps=2e-5,
              tie_word_embeddings=False, max_position_embeddings=2048)
# The layer shape of Llama 3.2 1B, which the benchmark runs, with 2 of its 16 layers: every product, the attention and the
# head at their real sizes (the plain model needs a few seconds for it; weights N(0, 0.02) keep scores and logits of order one).
LLAMA_1B_SHAPE = dict(hidden_size=2048, intermediate_size=8192, num_hidden_layers=2, num_attention_heads=32, num_key_value_heads=8,
                      head_dim=64, vocab_size=128256, rope_theta=500000.0,
                      rope_scaling=dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                        original_max_position_embeddings=8192),
                      rms_norm_eps=1e-5, tie_word_embeddings=True, max_position_embeddings=4096)
# The layer shape of Llama 3.2 3B (24 query heads over 8 key/value heads of 128 channels, hidden 3072) with one layer and a
# vocabulary cut to a number that is no multiple of anything: heads of 128 channels and widths that are no power of two in one model.
LLAMA_3B_SHAPE = dict(hidden_size=3072, intermediate_size=8192, num_hidden_layers=1, num_attention_heads=24, num_key_value_heads=8,
                      head_dim=128, vocab_size=32003, rope_theta=500000.0,
                      rope_scaling=dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                        original_max_position_embeddings=8192),
                      rms_norm_eps=1e-5, tie_word_embeddings=True, max_position_embeddings=4096)
PAGE_SIZE = {"A": 4, "B": 8, "C": 16, "D": 16}
CONFIGS = {"A": TINY_A, "B": TINY_B, "C": TINY_C, "D": TINY_D}


def full_config(sizes: dict) -> dict:
    return {"architectures": ["LlamaForCausalLM"], "model_type": "llama", "hidden_act": "silu", "attention_bias": False,
            "mlp_bias": False, **sizes}


def tensor_layout(cfg: dict):
    """Names and shapes of a Llama folder (src/loader/hf_checkpoint.cpp:214-235)."""
    d, i, v = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    heads = cfg["num_attention_heads"]
    kvh = cfg.get("num_key_value_heads") or heads
    hd = cfg.get("head_dim") or d // heads
    out = [("model.embed_tokens.weight", (v, d))]
    for l in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{l}."
        out += [(p + "input_layernorm.weight", (d,)), (p + "self_attn.q_proj.weight", (heads * hd, d)),
                (p + "self_attn.k_proj.weight", (kvh * hd, d)), (p + "self_attn.v_proj.weight", (kvh * hd, d)),
                (p + "self_attn.o_proj.weight", (d, heads * hd)), (p + "post_attention_layernorm.weight", (d,)),
                (p + "mlp.gate_proj.weight", (i, d)), (p + "mlp.up_proj.weight", (i, d)), (p + "mlp.down_proj.weight", (d, i))]
    out.append(("model.norm.weight", (d,)))
    if not cfg.get("tie_word_embeddings", False):
        out.append(("lm_head.weight", (v, d)))
    return out


def random_weights(cfg: dict, seed: int, std: float = 0.2):
    rng = np.random.default_rng(seed)
    w = {}
    for name, shape in tensor_layout(cfg):
        if name.endswith("norm.weight"):
            w[name] = torch.from_numpy((1.0 + 0.1 * rng.standard_normal(shape)).astype(np.float32))
        else:
            w[name] = torch.from_numpy((std * rng.standard_normal(shape)).astype(np.float32))
    return w


def formula_weights(cfg: dict, seed: int, std: float = 0.02):
    """The weights that the engine draws on the device for `seed` (`random_model(..., draw_on_device=True)`), re-made here from the
    formula its documentation states, in this file's own words: key = fnv1a64(name) + (seed + 1) * golden; element i (row-major)
    takes r = splitmix64's finaliser of key + (i + 1) * golden, u1 = ((r >> 40) + 1) / 2^24, u2 = ((r >> 8) & 0xFFFFFF) / 2^24,
    z = sqrt(-2 ln u1) cos(2 pi u2) in 64-bit; matrices std * z, norm weights 1 + 0.1 z, rounded to 32-bit."""
    golden, mask = 0x9E3779B97F4A7C15, (1 << 64) - 1
    out = {}
    for name, shape in tensor_layout(cfg):
        key = 0xCBF29CE484222325
        for byte in name.encode():
            key = ((key ^ byte) * 0x100000001B3) & mask
        key = (key + (seed + 1) * golden) & mask
        n = int(np.prod(shape))
        values = np.empty(n, dtype=np.float32)
        offset, scale = (1.0, 0.1) if name.endswith("norm.weight") else (0.0, std)
        with np.errstate(over="ignore"):
            for start in range(0, n, 1 << 24):
                i = np.arange(start + 1, min(n, start + (1 << 24)) + 1, dtype=np.uint64)
                z = np.uint64(key) + i * np.uint64(golden)
                z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
                z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
                z = z ^ (z >> np.uint64(31))
                u1 = ((z >> np.uint64(40)).astype(np.float64) + 1.0) / 2.0 ** 24
                u2 = ((z >> np.uint64(8)) & np.uint64(0xFFFFFF)).astype(np.float64) / 2.0 ** 24
                values[start:start + len(i)] = (offset + scale * (np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2))).astype(np.float32)
        out[name] = torch.from_numpy(values).reshape(shape)
    return out


_NAMES = {torch.float32: "F32", torch.bfloat16: "BF16", torch.float16: "F16", torch.int32: "I32", torch.int64: "I64", torch.float64: "F64"}


def write_safetensors_by_hand(path, tensors: dict, shuffle_seed=None, header_pad=0):
    names = list(tensors)
    if shuffle_seed is not None:
        np.random.default_rng(shuffle_seed).shuffle(names)
    header, blobs, off = {"__metadata__": {"format": "pt"}}, [], 0
    for n in names:
        t = tensors[n].contiguous()
        raw = t.reshape(-1).view(torch.uint8).numpy().tobytes()
        header[n] = {"dtype": _NAMES[t.dtype], "shape": list(t.shape), "data_offsets": [off, off + len(raw)]}
        off += len(raw)
        blobs.append(raw)
    text = json.dumps(header).encode() + b" " * header_pad
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(text)) + text)
        for raw in blobs:
            f.write(raw)


def write_model(folder, sizes: dict, seed: int = 0, dtype=torch.bfloat16, norm_dtype=None, std: float = 0.2, weights=None):
    """Writes the folder; returns the float32 weights before rounding to the storage dtype."""
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    cfg = full_config(sizes)
    (folder / "config.json").write_text(json.dumps(cfg, indent=2))
    w = weights if weights is not None else random_weights(cfg, seed, std)
    stored = {n: t.to(norm_dtype or dtype) if n.endswith("norm.weight") else t.to(dtype) for n, t in w.items()}
    write_safetensors_by_hand(folder / "model.safetensors", stored, shuffle_seed=seed + 17)
    return w


def relative_error(got, want) -> float:
    """max|got - want| / max|want|: stricter than the reference's measure, which floors the
    denominator at 1 (tests/verify_forward.py:72-77)."""
    got = torch.as_tensor(got).double().cpu()
    want = torch.as_tensor(want).double().cpu()
    return float((got - want).abs().max() / want.abs().max().clamp_min(1e-30))


def assert_within_bfloat16_noise(got: dict, exact, rounded, what=""):
    """The criterion for whole-model logits in bfloat16.

    `got[key]` are the engine's rows, `exact(key)` the 64-bit plain model's, `rounded(key)` those of the
    plain model that rounds to bfloat16 where the engine stores bfloat16.  One value that falls on the
    other side of a rounding edge changes everything after it by the size of the rounding noise, so the
    rounding plain model is no tighter a reference than the exact one; what can be asked is that the
    engine is as close to the exact model as rounding alone explains: its mean error within 1.5x and
    its worst error within 2x of the rounding plain model's.  A fault of masking, paging or order shows
    as errors many times the noise."""
    errors = [relative_error(row, exact(key)) for key, row in got.items()]
    noise = [relative_error(rounded(key), exact(key)) for key in got]
    mean_e, mean_n = sum(errors) / len(errors), sum(noise) / len(noise)
    assert mean_e < 1.5 * mean_n + 1e-4, f"{what}: mean error {mean_e:.3e} against rounding noise {mean_n:.3e}"
    assert max(errors) < 2.0 * max(noise) + 1e-4, f"{what}: worst error {max(errors):.3e} against rounding noise {max(noise):.3e}"
    return mean_e, mean_n
