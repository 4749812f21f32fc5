"""What pins the plain implementation beside the reference's text: special cases that reduce to a
library routine, other formulations of the same formula, and invariants, each chosen so that a
plausible mistake fails it.  The engine's own host-side formulas are held against the plain ones."""
import math

import numpy as np
import pytest
import torch

import plain_sampler
from plain_llama import (PlainLlama, causal_attention, rms_norm, rope_inverse_frequencies, rope_rotate, swiglu)
from model_folders import CONFIGS, write_model

torch.manual_seed(0)


# ------------------------------------------------------------------------------------------ norm
def test_rms_norm_with_unit_weight_is_x_over_rms():
    x = torch.randn(5, 37, dtype=torch.float64)
    for eps in (1e-6, 0.05):                                         # a large eps shows an eps outside the root (tests/verify_forward.py:53)
        want = x / torch.sqrt((x ** 2).mean(-1, keepdim=True) + eps)
        assert torch.allclose(rms_norm(x, torch.ones(37, dtype=torch.float64), eps), want, atol=1e-14)
    w = torch.randn(37, dtype=torch.float64)
    assert torch.allclose(rms_norm(x, w, 1e-5), w * rms_norm(x, torch.ones(37, dtype=torch.float64), 1e-5))   # the weight as it is, not 1 + w
    assert torch.isfinite(rms_norm(torch.zeros(2, 8, dtype=torch.float64), torch.ones(8, dtype=torch.float64), 1e-6)).all()


# ------------------------------------------------------------------------------------------ rope
def rotate_half_form(x, positions, inv_freq):
    """x*cos + rotate_half(x)*sin with cos/sin doubled over both halves (tests/verify_kernels.py:284-291)."""
    hd = x.shape[-1]
    ang = positions.double()[:, None] * inv_freq[None, :]
    cos, sin = torch.cat([ang.cos(), ang.cos()], -1)[:, None, :], torch.cat([ang.sin(), ang.sin()], -1)[:, None, :]
    return x * cos + torch.cat([-x[..., hd // 2:], x[..., :hd // 2]], -1) * sin


def test_rope_is_the_rotate_half_statement():
    for hd, theta in ((16, 10000.0), (64, 100000.0), (32, 500000.0)):
        x = torch.randn(7, 3, hd, dtype=torch.float64)
        pos = torch.tensor([0, 1, 9, 100, 2047, 8191, 31999])
        inv = rope_inverse_frequencies(hd, theta)
        got = rope_rotate(x, pos, inv)
        assert torch.allclose(got, rotate_half_form(x, pos, inv), atol=1e-12)
        assert torch.equal(got[0], x[0])                             # position 0 is the identity
        n_in = x[..., :hd // 2] ** 2 + x[..., hd // 2:] ** 2         # every pair keeps its length
        n_out = got[..., :hd // 2] ** 2 + got[..., hd // 2:] ** 2
        assert torch.allclose(n_in, n_out, atol=1e-12)
        interleaved = x.clone()                                      # the other pairing gives something else
        a, b = x[..., 0::2], x[..., 1::2]
        ang = pos.double()[:, None, None] * inv[None, None, :]
        interleaved[..., 0::2], interleaved[..., 1::2] = a * ang.cos() - b * ang.sin(), a * ang.sin() + b * ang.cos()
        assert not torch.allclose(got[2:], interleaved[2:], atol=1e-3)


LLAMA3_CASES = [  # theta, factor, low, high, original, head size (tests/verify_kernels.py:319-325)
    (500000.0, 32.0, 1.0, 4.0, 8192, 64), (500000.0, 8.0, 1.0, 4.0, 8192, 128), (500000.0, 4.0, 1.0, 4.0, 64, 16),
    (10000.0, 2.0, 0.5, 6.0, 100, 32), (100000.0, 16.0, 1.0, 2.0, 37, 8),
]


@pytest.mark.parametrize("theta,factor,low,high,original,hd", LLAMA3_CASES)
def test_llama3_frequencies_in_another_formulation(theta, factor, low, high, original, hd):
    """The vectorised statement of tools/ref.py:36-51 (np.where over wavelengths) against the loop."""
    scaling = dict(factor=factor, low_freq_factor=low, high_freq_factor=high, original_max_position_embeddings=original)
    freqs = 1.0 / (theta ** (np.arange(0, hd, 2, dtype=np.float64) / hd))
    wavelen = 2 * np.pi / freqs
    scaled = np.where(wavelen > original / low, freqs / factor, freqs)
    smooth = (original / wavelen - low) / (high - low)
    smoothed = (1 - smooth) * scaled / factor + smooth * scaled
    medium = ~(wavelen < original / high) & ~(wavelen > original / low)
    want = np.where(medium, smoothed, scaled)
    got = rope_inverse_frequencies(hd, theta, scaling).numpy()
    assert np.allclose(got, want, rtol=1e-14)
    assert np.any(got == freqs) or np.any(np.isclose(got, freqs / factor))          # some frequency is unscaled or fully stretched
    assert not np.allclose(got, freqs)                                               # and scaling changes something


def test_the_engine_computes_the_same_frequencies():
    from geneinfer_amd.config import Llama3Scaling
    from geneinfer_amd.config.llama import rotary_frequencies
    from geneinfer_amd.parts.rope import inverse_frequencies
    for theta, factor, low, high, original, hd in LLAMA3_CASES:
        got = rotary_frequencies(hd, theta, Llama3Scaling(factor, low, high, original))
        want = rope_inverse_frequencies(hd, theta, dict(factor=factor, low_freq_factor=low, high_freq_factor=high,
                                                        original_max_position_embeddings=original))
        assert np.allclose(got, want.numpy(), rtol=1e-15)
    assert np.allclose(inverse_frequencies(32, 10000.0), rope_inverse_frequencies(32, 10000.0).numpy(), rtol=1e-15)


def test_scores_depend_on_distance_only():
    """Shifting all positions leaves q.k unchanged: a wrong sign in the rotation breaks this."""
    hd = 32
    inv = rope_inverse_frequencies(hd, 500000.0, dict(factor=4, low_freq_factor=1, high_freq_factor=4, original_max_position_embeddings=32))
    q, k = torch.randn(1, 1, hd, dtype=torch.float64), torch.randn(1, 1, hd, dtype=torch.float64)
    def score(pq, pk):
        return float((rope_rotate(q, torch.tensor([pq]), inv) * rope_rotate(k, torch.tensor([pk]), inv)).sum())
    assert abs(score(10, 3) - score(110, 103)) < 1e-10 and abs(score(10, 3) - score(1007, 1000)) < 1e-9
    assert abs(score(10, 3) - score(3, 10)) > 1e-3                   # but the direction matters


# ------------------------------------------------------------------------------------- attention
def test_attention_with_equal_head_counts_is_the_library_routine():
    T, H, hd = 11, 3, 16
    q, k, v = (torch.randn(T, H, hd, dtype=torch.float64) for _ in range(3))
    want = torch.nn.functional.scaled_dot_product_attention(q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True).transpose(0, 1)
    assert torch.allclose(causal_attention(q, k, v), want, atol=1e-12)


def test_grouped_heads_are_repeated_key_value_heads():
    T, H, KV, hd = 9, 6, 2, 8
    q = torch.randn(T, H, hd, dtype=torch.float64)
    k, v = torch.randn(T, KV, hd, dtype=torch.float64), torch.randn(T, KV, hd, dtype=torch.float64)
    want = causal_attention(q, k.repeat_interleave(H // KV, 1), v.repeat_interleave(H // KV, 1))
    assert torch.allclose(causal_attention(q, k, v), want, atol=1e-14)
    assert not torch.allclose(causal_attention(q, k, v), causal_attention(q, k.repeat(1, H // KV, 1), v.repeat(1, H // KV, 1)))   # h // G, not h % KV


def test_attention_special_cases():
    hd = 8
    q, k, v = (torch.randn(5, 2, hd, dtype=torch.float64) for _ in range(3))
    out = causal_attention(q, k, v)
    assert torch.allclose(out[0], v[0])                              # one position: the softmax of one score is 1
    flat = causal_attention(torch.zeros_like(q), k, v)
    assert torch.allclose(flat[3], v[:4].mean(0))                    # equal scores: the mean of what is visible
    big = causal_attention(q * 300, k, v)
    assert torch.isfinite(big).all()                                 # scores near 1000 do not overflow
    win = causal_attention(q, k, v, window=2)
    assert torch.allclose(win[4], causal_attention(q[3:], k[3:], v[3:])[1])          # row 4 sees rows 3 and 4 only
    assert torch.allclose(win[1], out[1])


# ----------------------------------------------------------------------------------- feed-forward
def test_swiglu_is_silu_times_up():
    x = torch.randn(4, 12, dtype=torch.float64) * 5
    wg, wu, wd = torch.randn(20, 12, dtype=torch.float64), torch.randn(20, 12, dtype=torch.float64), torch.randn(12, 20, dtype=torch.float64)
    want = (torch.nn.functional.silu(x @ wg.T) * (x @ wu.T)) @ wd.T
    assert torch.allclose(swiglu(x, wg, wu, wd), want, atol=1e-10)


# ------------------------------------------------------------------------------------ whole model
def test_whole_model_properties(tmp_path):
    write_model(tmp_path, CONFIGS["B"], seed=3, dtype=torch.float32)
    m = PlainLlama(tmp_path)
    toks = [5, 99, 201, 17, 300, 42]
    full = m.logits(toks)
    assert torch.allclose(m.logits(toks[:4]), full[:4], atol=1e-12)  # causal: a prefix gives the same logits
    other = m.logits([6] + toks[1:])
    assert float((other[-1] - full[-1]).abs().max()) > 1e-3          # the first token matters
    w = dict(m.w)                                                    # position 0 does not depend on wq or wk
    m.w = {k: (torch.randn_like(v) if "q_proj" in k or "k_proj" in k else v) for k, v in w.items()}
    assert torch.allclose(m.logits(toks)[0], full[0], atol=1e-12) and not torch.allclose(m.logits(toks)[1], full[1], atol=1e-6)
    m.w = w
    assert not torch.equal(m.w["lm_head.weight"], m.w["model.embed_tokens.weight"])    # B is untied: its own head is used
    head = m.w["lm_head.weight"]
    m.w = {**w, "lm_head.weight": head * 2}
    assert torch.allclose(m.logits(toks), 2 * full, atol=1e-10)


def test_bfloat16_storage_rounds_but_stays_close(tmp_path):
    write_model(tmp_path, CONFIGS["A"], seed=3, dtype=torch.bfloat16)
    toks = list(range(10, 40))
    exact, rounded = PlainLlama(tmp_path).logits(toks), PlainLlama(tmp_path, storage=torch.bfloat16).logits(toks)
    err = float((exact - rounded).abs().max() / exact.abs().max())
    assert 1e-4 < err < 0.1


# ---------------------------------------------------------------------------------------- sampler
def test_greedy_takes_the_lowest_index_among_equals():              # tests/verify_sampler.py:173-178
    for logits, want in (([1, 5, 5, 2], 1), ([3, 3, 3], 0), ([-7], 0), ([0, -1, 9, 9, 9, 4], 2)):
        assert plain_sampler.sample(logits, 0.0, 5, 0.5, 0.7) == want


def test_uniform_stream_properties():
    u = plain_sampler.uniforms(7, 20000)
    assert u.min() >= 0.0 and u.max() < 1.0 and abs(u.mean() - 0.5) < 0.01
    assert np.array_equal(plain_sampler.uniforms(0, 5), plain_sampler.uniforms(0, 5))
    assert not np.array_equal(plain_sampler.uniforms(5, 50), plain_sampler.uniforms(6, 50))
    assert np.all(u * 16777216.0 == np.floor(u * 16777216.0))        # 24 random bits


def test_filters_keep_what_they_should():
    flat = np.zeros(10, dtype=np.float32)                            # all ties: lowest indices first (tests/verify_sampler.py:161-166)
    rng = np.random.default_rng(0)
    us = rng.random(300, dtype=np.float32)
    assert {plain_sampler.sample(flat, 1.0, 3, 1.0, u) for u in us} == {0, 1, 2}
    assert {plain_sampler.sample(flat, 1.0, 0, 0.35, u) for u in us} == {0, 1, 2, 3}
    peaked = np.zeros(20, dtype=np.float32)
    peaked[13] = 30.0
    assert {plain_sampler.sample(peaked, 1.0, 0, 0.9, u) for u in us} == {13}
    logits = np.array([2.0, 1.0, 0.5, 0.0, -1.0, -3.0], dtype=np.float32)
    p = np.exp(logits.astype(np.float64)) / np.exp(logits.astype(np.float64)).sum()
    draws = np.array([plain_sampler.sample(logits, 1.0, 0, 1.0, u) for u in plain_sampler.uniforms(99, 30000)])
    for tok in range(6):                                             # frequencies within five sigma (tests/verify_sampler.py:181-200)
        z = (np.sum(draws == tok) - 30000 * p[tok]) / math.sqrt(30000 * p[tok] * (1 - p[tok]))
        assert abs(z) < 5


def test_the_engine_samples_as_the_plain_sampler():
    from geneinfer_amd.sampling import SamplerConfig, UniformStream, filtered_draw
    for seed in (0, 1, 42, 2 ** 63 + 12345):
        s = UniformStream(seed)
        assert np.array_equal(np.array([s.next_uniform() for _ in range(500)], dtype=np.float32), plain_sampler.uniforms(seed, 500))
    rng = np.random.default_rng(1)
    for vocab in (2, 5, 100, 4000):
        logits = (2 * rng.standard_normal(vocab)).astype(np.float32)
        for t, k, p in [(0.3, 0, 1.0), (1.0, 0, 0.9), (0.8, 0, 0.5), (1.0, 0, 0.05), (1.0, 3, 1.0), (1.5, 50, 1.0), (1.0, 5, 0.9), (0.7, 1, 1.0),
                        (1.0, 1000000, 1.0), (1.0, 4, 0.3)]:
            for u in list(rng.random(40, dtype=np.float32)) + [0.0, 0.5, np.float32(1.0 - 2.0 ** -24)]:
                assert filtered_draw(logits, SamplerConfig(t, k, p, 1), float(u)) == plain_sampler.sample(logits, t, k, p, u)
    with pytest.raises(ValueError):
        SamplerConfig(temperature=-1.0).validate(10)
    for bad in (SamplerConfig(top_k=-1), SamplerConfig(top_p=0.0), SamplerConfig(top_p=1.5), SamplerConfig(temperature=float("nan"))):
        with pytest.raises(ValueError):
            bad.validate(10)
    with pytest.raises(ValueError):
        SamplerConfig().validate(0)
