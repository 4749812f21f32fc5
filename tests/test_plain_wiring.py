"""Pins of the plain model that are not a second reading of the same text: the llama3 change of frequencies held to
values worked out by hand and to the shape it must have, and the wiring of a block (norm before each half, two
residual sums, the final norm) held to special cases that reduce to library routines and to a whole forward pass
composed of library routines only (torch.nn.functional's rms_norm, linear, silu and scaled_dot_product_attention,
the rotation as a complex product).  A post-norm block, a missing residual, a norm in the wrong place, a wrong
pairing or sign of the rotation, a head taken modulo instead of divided, or swapped branches of the scaling each
fail one of them.  (Model code of installed packages is not used here or anywhere: it is no source for this build.)"""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from model_folders import CONFIGS, full_config, random_weights, write_model
from plain_llama import PlainLlama, rope_inverse_frequencies

from test_plain import LLAMA3_CASES


# ------------------------------------------------------------------------------- llama3 scaling
def test_llama3_frequencies_of_tiny_b_by_hand():
    """hd 32, theta 5e5, factor 4, low 1, high 4, original 32.  Wavelengths 2*pi*theta^(k/16): 6.28 (below 32/4 = 8:
    kept), 14.27 (between 8 and 32: blended), 32.4 and longer (above 32/1: divided by 4).  tests/verify_forward.py:64
    runs the same three regimes in one head."""
    sc = CONFIGS["B"]["rope_scaling"]
    got = rope_inverse_frequencies(32, 5e5, sc).tolist()
    plain = [5e5 ** (-k / 16.0) for k in range(16)]
    assert got[0] == 1.0
    wavelength = 2 * math.pi * 5e5 ** (1 / 16.0)
    assert 14.2 < wavelength < 14.3
    smooth = (32.0 / wavelength - 1.0) / 3.0
    assert 0.41 < smooth < 0.42
    assert got[1] == pytest.approx(plain[1] * (0.25 * (1 - smooth) + smooth), rel=1e-14) and plain[1] / 4 < got[1] < plain[1]
    assert 2 * math.pi / plain[2] > 32.0
    for k in range(2, 16):
        assert got[k] == pytest.approx(plain[k] / 4.0, rel=1e-14)          # (the power is taken in two ways: units in the last place)


@pytest.mark.parametrize("theta,factor,low,high,original,hd", LLAMA3_CASES)
def test_llama3_scaling_keeps_fast_turns_and_slows_slow_ones(theta, factor, low, high, original, hd):
    """got / plain falls from 1 (short wavelengths) to 1 / factor (long ones) and never rises with k; exactly 1 below
    original / high, exactly 1 / factor above original / low.  With the two outer branches swapped the ratio would rise."""
    scaling = dict(factor=factor, low_freq_factor=low, high_freq_factor=high, original_max_position_embeddings=original)
    got = rope_inverse_frequencies(hd, theta, scaling).numpy()
    plain = rope_inverse_frequencies(hd, theta).numpy()
    ratio = got / plain
    wavelength = 2 * np.pi / plain
    assert np.all(np.diff(ratio) <= 1e-15) and ratio[0] == 1.0 and ratio[-1] == pytest.approx(1 / factor, rel=1e-15)
    assert np.all(ratio[wavelength < original / high] == 1.0)
    assert np.allclose(ratio[wavelength > original / low], 1 / factor, rtol=1e-15)
    between = (wavelength >= original / high) & (wavelength <= original / low)
    assert np.all((ratio[between] <= 1.0) & (ratio[between] >= 1 / factor - 1e-15))


# ---------------------------------------------------------------------- a forward pass of library routines
def library_forward(cfg, w, tokens, inv_freq):
    """The decoder over one sequence with library routines only.  The rotation is the complex product
    (a + i b) * exp(i * pos * f_k) of the pair a = x[k], b = x[k + head_dim/2]."""
    w = {k: v.double() for k, v in w.items()}
    H, hd = cfg["num_attention_heads"], cfg.get("head_dim") or cfg["hidden_size"] // cfg["num_attention_heads"]
    KV, eps, T = cfg.get("num_key_value_heads") or H, cfg["rms_norm_eps"], len(tokens)
    turn = torch.polar(torch.ones(T, hd // 2, dtype=torch.float64), torch.arange(T, dtype=torch.float64)[:, None] * inv_freq[None, :])

    def rotate(x):                                                  # [T, heads, hd]
        z = torch.complex(x[..., :hd // 2], x[..., hd // 2:]) * turn[:, None, :]
        return torch.cat([z.real, z.imag], dim=-1)

    x = F.embedding(torch.tensor(tokens), w["model.embed_tokens.weight"])
    for l in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{l}."
        h = F.rms_norm(x, (x.shape[-1],), w[p + "input_layernorm.weight"], eps)
        q = rotate(F.linear(h, w[p + "self_attn.q_proj.weight"]).view(T, H, hd)).transpose(0, 1)
        k = rotate(F.linear(h, w[p + "self_attn.k_proj.weight"]).view(T, KV, hd)).transpose(0, 1)
        v = F.linear(h, w[p + "self_attn.v_proj.weight"]).view(T, KV, hd).transpose(0, 1)
        att = F.scaled_dot_product_attention(q[None], k[None], v[None], is_causal=True, enable_gqa=True)[0]
        x = x + F.linear(att.transpose(0, 1).reshape(T, H * hd), w[p + "self_attn.o_proj.weight"])
        h = F.rms_norm(x, (x.shape[-1],), w[p + "post_attention_layernorm.weight"], eps)
        x = x + F.linear(F.silu(F.linear(h, w[p + "mlp.gate_proj.weight"])) * F.linear(h, w[p + "mlp.up_proj.weight"]), w[p + "mlp.down_proj.weight"])
    x = F.rms_norm(x, (x.shape[-1],), w["model.norm.weight"], eps)
    head = w["model.embed_tokens.weight"] if cfg.get("tie_word_embeddings") else w["lm_head.weight"]
    return F.linear(x, head)


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_plain_model_is_the_composition_of_library_routines(name, tmp_path):
    cfg = CONFIGS[name]
    w = write_model(tmp_path, cfg, seed=21, dtype=torch.float32)
    plain = PlainLlama(tmp_path)
    rng = np.random.default_rng(1)
    tokens = rng.integers(0, cfg["vocab_size"], 50).tolist()        # past tiny B's original context of 32
    want = library_forward(full_config(cfg), w, tokens, plain.inv_freq)
    got = plain.logits(tokens)
    assert float((got - want).abs().max() / want.abs().max()) < 1e-12


# ----------------------------------------------------------------------------- wiring special cases
def silenced(cfg, seed, which):
    w = random_weights(full_config(cfg), seed)
    for n in w:
        if any(n.endswith(s) for s in which):
            w[n] = torch.zeros_like(w[n])
    return w


def test_with_silent_halves_the_logits_are_the_head_of_the_normed_embedding(tmp_path):
    """o_proj = down_proj = 0 in every layer: each half adds nothing, the residual stream stays the embedding, and the
    logits are head(rms_norm(embedding)).  A block that norms the stream itself (post-norm) or drops the residual fails."""
    cfg = CONFIGS["B"]
    w = silenced(cfg, 5, ("o_proj.weight", "down_proj.weight"))
    write_model(tmp_path, cfg, dtype=torch.float32, weights=w)
    tokens = [3, 200, 77, 9, 310]
    e = w["model.embed_tokens.weight"].double()[torch.tensor(tokens)]
    want = F.linear(F.rms_norm(e, (e.shape[-1],), w["model.norm.weight"].double(), cfg["rms_norm_eps"]), w["lm_head.weight"].double())
    assert torch.allclose(PlainLlama(tmp_path).logits(tokens), want, atol=1e-12)


def test_one_token_through_one_layer_in_closed_form(tmp_path):
    """One token at position 0: the rotation is the identity and the softmax of one score is 1, so attention gives each
    query head the value head of its group.  x1 = e + Wo * repeat(Wv * norm1(e)); x2 = x1 + W2 (silu(W1 n) * W3 n) with
    n = norm2(x1); logits = head(norm_f(x2)).  Checks both residual sums, the three norms' places and the grouping h // G."""
    cfg = dict(CONFIGS["C"])                                        # one layer, 6 heads over 3 value heads
    w = write_model(tmp_path, cfg, seed=8, dtype=torch.float32)
    d = {k: v.double() for k, v in w.items()}
    p, eps = "model.layers.0.", cfg["rms_norm_eps"]
    H, KV, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["head_dim"]
    token = 123
    e = d["model.embed_tokens.weight"][token]
    n1 = F.rms_norm(e, (e.shape[0],), d[p + "input_layernorm.weight"], eps)
    v = (d[p + "self_attn.v_proj.weight"] @ n1).view(KV, hd)
    x1 = e + d[p + "self_attn.o_proj.weight"] @ v.repeat_interleave(H // KV, dim=0).reshape(H * hd)
    n2 = F.rms_norm(x1, (e.shape[0],), d[p + "post_attention_layernorm.weight"], eps)
    x2 = x1 + d[p + "mlp.down_proj.weight"] @ (F.silu(d[p + "mlp.gate_proj.weight"] @ n2) * (d[p + "mlp.up_proj.weight"] @ n2))
    want = d["lm_head.weight"] @ F.rms_norm(x2, (e.shape[0],), d["model.norm.weight"], eps)
    got = PlainLlama(tmp_path).logits([token])[0]
    assert torch.allclose(got, want, atol=1e-12)
    wrong_groups = e + d[p + "self_attn.o_proj.weight"] @ v.repeat(H // KV, 1).reshape(H * hd)       # h % KV instead of h // G
    assert not torch.allclose(x1, wrong_groups, atol=1e-6)
