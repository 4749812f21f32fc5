"""Each kernel alone against a plain torch statement of the same operation, at sizes other than
the engine's test models: primes, sizes that are no multiple of a tile, single rows."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def ops():
    from geneinfer_amd.kernels import ops as o
    return o


def rel(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    return float((got - want).abs().max() / want.abs().max().clamp_min(1e-30))


def randn(*shape, dtype=torch.float32, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed + sum(shape))
    return (scale * torch.randn(*shape, generator=g)).to(dtype).to(DEV)


# ------------------------------------------------------------------------------------------ gemm
@pytest.mark.parametrize("m,n,k", [(1, 1, 1), (1, 7, 13), (5, 64, 64), (64, 65, 17), (130, 257, 96), (3, 1000, 515)])
@pytest.mark.parametrize("dtypes", [(torch.float32, torch.float32), (torch.float32, torch.bfloat16), (torch.bfloat16, torch.bfloat16)])
def test_gemm_exact(m, n, k, dtypes):
    a, w = randn(m, k, dtype=dtypes[0], seed=1), randn(n, k, dtype=dtypes[1], seed=2)
    out = torch.full((m, n + 3), -777.25, device=DEV)                 # a wider output keeps its rim
    ops().gemm_exact(a, w, out[:, :n])
    want = a.double() @ w.double().T
    assert rel(out[:, :n], want) < 2e-6
    assert torch.all(out[:, n:] == -777.25)
    before = out[:, :n].clone()
    ops().gemm_exact(a, w, out[:, :n], accumulate=True)
    assert rel(out[:, :n], 2 * want) < 2e-6 and not torch.equal(before, out[:, :n])


def test_gemm_exact_rows_alone_have_the_same_bits():
    a, w = randn(37, 200, seed=3), randn(90, 200, seed=4)
    full = torch.empty(37, 90, device=DEV)
    ops().gemm_exact(a, w, full)
    for i in (0, 17, 36):
        one = torch.empty(1, 90, device=DEV)
        ops().gemm_exact(a[i:i + 1], w, one)
        assert torch.equal(one[0], full[i])


@pytest.mark.parametrize("m,n,k", [(1, 16, 8), (1, 2048, 2048), (3, 100, 136), (8, 130, 264), (16, 64, 128), (17, 1000, 520),
                                   (33, 48, 72), (64, 515, 1032), (65, 128, 64), (100, 300, 200), (128, 128, 128), (200, 257, 96),
                                   (513, 384, 1024), (2048, 96, 160)])
@pytest.mark.parametrize("out_dtype,accumulate", [(torch.float32, False), (torch.float32, True), (torch.bfloat16, False)])
def test_gemm_bf16(m, n, k, out_dtype, accumulate):
    a, w = randn(m, k, dtype=torch.bfloat16, seed=5), randn(n, k, dtype=torch.bfloat16, seed=6)
    base = randn(m, n + 5, seed=7).to(out_dtype)
    out = base.clone()
    ops().gemm_bf16(a, w, out[:, :n], accumulate=accumulate)
    want = a.double() @ w.double().T + (base[:, :n].double() if accumulate else 0)
    tol = 1e-5 if out_dtype == torch.float32 else 5e-3
    assert rel(out[:, :n], want) < tol, (m, n, k)
    assert torch.equal(out[:, n:], base[:, n:])


def test_gemm_bf16_refuses_what_it_cannot_do():
    o = ops()
    a, w = randn(4, 12, dtype=torch.bfloat16), randn(6, 12, dtype=torch.bfloat16)
    out = torch.empty(4, 6, device=DEV)
    assert not o.gemm_bf16_supports(a, w, out)                       # K = 12 is no multiple of 8
    with pytest.raises(o.KernelError):
        o.gemm_bf16(a, w, out)


# ------------------------------------------------------------------------------- row-wise kernels
@pytest.mark.parametrize("n,dim", [(1, 1), (3, 17), (5, 256), (2, 1000), (7, 4099)])
@pytest.mark.parametrize("w_dtype,out_dtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16), (torch.float32, torch.bfloat16)])
def test_rmsnorm(n, dim, w_dtype, out_dtype):
    x, w = randn(n, dim, seed=8, scale=3.0), (1 + 0.1 * randn(dim, seed=9)).to(w_dtype)
    for eps in (1e-6, 0.05):                                         # a large eps shows an eps in the wrong place
        out = torch.empty(n, dim, dtype=out_dtype, device=DEV)
        ops().rmsnorm(x, w, eps, out)
        xd = x.double()
        want = w.double() * (xd / torch.sqrt((xd * xd).mean(-1, keepdim=True) + eps))
        assert rel(out, want) < (2e-6 if out_dtype == torch.float32 else 5e-3)
    zero = torch.zeros(1, dim, device=DEV)
    out = torch.empty(1, dim, device=DEV)
    ops().rmsnorm(zero, w.float(), 1e-6, out)
    assert torch.isfinite(out).all() and float(out.abs().max()) == 0.0


def test_embed_and_gather():
    table = randn(50, 24, dtype=torch.bfloat16, seed=10)
    toks = torch.tensor([3, 49, 0, 3], dtype=torch.int32, device=DEV)
    out = torch.empty(4, 24, device=DEV)
    ops().embed(table, toks, out)
    assert torch.equal(out, table[toks.long()].float())
    picked = torch.empty(2, 24, device=DEV)
    ops().gather_rows(out, torch.tensor([2, 1], dtype=torch.int32, device=DEV), picked)
    assert torch.equal(picked, out[[2, 1]])


def test_silu_mul():
    gu = randn(5, 2 * 37, seed=11, scale=4.0)
    gu[0, 0], gu[0, 1] = 100.0, -100.0                               # extremes stay finite
    out = torch.empty(5, 37, device=DEV)
    ops().silu_mul(gu, out)
    want = torch.nn.functional.silu(gu[:, :37].double()) * gu[:, 37:].double()
    assert rel(out, want) < 2e-6 and torch.isfinite(out).all()


def test_rope_cos_sin_uses_64_bit_angles():
    pos = torch.tensor([0, 1, 4095, 131071, 2 ** 24 + 1], dtype=torch.int32, device=DEV)
    inv = torch.tensor([1.0, 0.3, 1e-3], dtype=torch.float64, device=DEV)
    cos, sin = torch.empty(5, 3, device=DEV), torch.empty(5, 3, device=DEV)
    ops().rope_cos_sin(pos, inv, cos, sin)
    ang = pos.double()[:, None] * inv[None, :]
    assert (cos.double() - torch.cos(ang)).abs().max() < 1e-7 and (sin.double() - torch.sin(ang)).abs().max() < 1e-7


# -------------------------------------------------------------------------------------- sampling
def test_argmax_lowest_index_on_ties():
    rows = [[1, 5, 5, 2], [3, 3, 3, 3], [-7, -8, -9, -10], [0, -1, 9, 9]]          # tests/verify_sampler.py:173-178
    logits = torch.tensor(rows, dtype=torch.float32, device=DEV)
    out = torch.empty(4, dtype=torch.int32, device=DEV)
    ops().argmax(logits, out)
    assert out.tolist() == [1, 0, 0, 2]
    big = randn(3, 128256, seed=12)
    big[1, 70000] = big[1, 5] = 50.0
    out = torch.empty(3, dtype=torch.int32, device=DEV)
    ops().argmax(big, out)
    assert out.tolist() == [int(torch.argmax(big[0])), 5, int(torch.argmax(big[2]))]


def test_sample_temperature_matches_the_inverse_distribution():
    import numpy as np
    from plain_sampler import sample
    g = torch.Generator().manual_seed(0)
    for vocab in (2, 5, 100, 3001, 128256):
        logits = (2 * torch.randn(8, vocab, generator=g)).float()
        temps = torch.tensor([0.3, 1.0, 2.0, 0.8, 1.0, 0.01, 1.5, 0.7])
        us = torch.cat([torch.rand(5, generator=g), torch.tensor([0.0, 0.5, 1.0 - 2.0 ** -24])]).float()
        out = torch.empty(8, dtype=torch.int32, device=DEV)
        ops().sample_temperature(logits.to(DEV), temps.to(DEV), us.to(DEV), out)
        for i, got in enumerate(out.tolist()):
            want = sample(logits[i].numpy(), float(temps[i]), 0, 1.0, float(us[i]))
            if got != want:                                          # only a draw on the edge between two tokens may differ
                p = torch.softmax(logits[i].double() / float(temps[i]), 0)
                cum = torch.cumsum(p, 0)
                assert abs(got - want) == 1 and float((cum - float(us[i])).abs().min()) < 1e-6, (vocab, i, got, want)
