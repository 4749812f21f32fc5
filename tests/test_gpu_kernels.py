"""Each kernel alone against a plain torch statement of the same operation, at sizes other than
the engine's test models: primes, sizes that are no multiple of a tile, single rows."""
import math

import numpy as np
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


@pytest.mark.parametrize("w_dtype,k", [(torch.float32, 200), (torch.float32, 203), (torch.bfloat16, 264), (torch.bfloat16, 520)])
def test_gemm_exact_rows_alone_have_the_same_bits(w_dtype, k):
    """One to four rows take the kernel with a lane per output column, more rows the tiled one; k = 203 leaves a tail
    beside the 16-byte loads, 264 and 520 pieces of 8 beside whole groups of 64."""
    a, w = randn(37, k, seed=3), randn(90, -(-k // 8) * 8, dtype=w_dtype, seed=4)[:, :k]      # the row stride stays a multiple of the 16-byte piece
    full = torch.empty(37, 90, device=DEV)
    ops().gemm_exact(a, w, full)
    for first, rows in ((0, 1), (17, 1), (36, 1), (5, 2), (9, 3), (30, 4)):
        few = torch.empty(rows, 90, device=DEV)
        ops().gemm_exact(a[first:first + rows], w, few)
        assert torch.equal(few, full[first:first + rows])
        ops().gemm_exact(a[first:first + rows], w, few, accumulate=True)
        both = full[first:first + rows].clone()
        ops().gemm_exact(a[first:first + rows].repeat(17, 1)[:rows + 13], w, (wide := torch.cat([both, torch.zeros(13, 90, device=DEV)])), accumulate=True)
        assert torch.equal(few, wide[:rows])                                # adding onto what is there, the same in both kernels


@pytest.mark.parametrize("m,n,k", [(1, 16, 8), (1, 2048, 2048), (3, 100, 136), (8, 130, 264), (16, 64, 128), (17, 1000, 520),
                                   (33, 48, 72), (64, 515, 1032), (65, 128, 64), (100, 300, 200), (128, 128, 128), (200, 257, 96),
                                   (513, 384, 1024), (2048, 96, 160),
                                   # the LDS-ring kernel: one block of k, edge tiles, each of its three tile choices
                                   (256, 160, 64), (130, 129, 192), (2100, 2200, 192), (4000, 8200, 128),
                                   # the ping-pong kernel (256 x 256 tiles for every compute unit or more): one block of k, an odd number of them, edges
                                   (4100, 4104, 64), (4096, 4100, 320),
                                   # ... with tiles for three quarters of the compute units only (3 x 64, and 3 x 65 with an edge on both sides)
                                   (768, 16384, 64), (520, 16400, 192),
                                   # ... and with k shared out over workgroups because the tiles are few
                                   (200, 256, 1024), (300, 2048, 2048), (129, 130, 512),
                                   # 65 to 128 rows: the skinny kernel with six or eight tiles of rows, narrow outputs (k shared out) and wide ones
                                   (72, 256, 1024), (65, 130, 512), (72, 2048, 2048), (96, 3072, 2048), (128, 2048, 8192), (80, 12300, 264), (113, 12288, 520),
                                   # wide outputs finished by the skinny kernel itself, from 12 rows and from 5
                                   (12, 12300, 520), (40, 12300, 264), (5, 65600, 72), (16, 12288, 256),
                                   # 17 to 32 rows, narrow outputs, short k: the slim kernel with two tiles of rows
                                   (32, 2048, 2048), (20, 3072, 2048), (31, 130, 136), (17, 16, 8),
                                   # up to 8 rows and a narrow output: the idle halves of the matrix instructions take a further 32 of k (blocks of 256, cut anywhere)
                                   (8, 2048, 8192), (4, 3072, 2048), (2, 3072, 264), (6, 1000, 1000), (7, 60, 8200), (8, 8, 32), (5, 24, 40),
                                   # ... and 9 to 16 rows, in two groups of 8 that share the weights
                                   (12, 2048, 8192), (9, 100, 136), (16, 3072, 2048), (13, 1000, 1000), (16, 8, 32),
                                   # strips of 12 or 8 weight rows that fill the compute units evenly, the last strip ragged (up to 16 rows, and 17 to 32)
                                   (13, 3000, 264), (8, 3071, 264), (3, 3072, 2048), (20, 2000, 264), (32, 2920, 2048)])
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


@pytest.mark.parametrize("m,inter,k", [(1, 16, 8), (5, 48, 136), (16, 160, 96), (17, 176, 64), (64, 32, 264), (70, 192, 128), (300, 8192 // 16, 2048 // 8),
                                       (72, 8192, 2048), (128, 6144, 264), (100, 288, 136),
                                       (40, 6144, 264), (13, 6160, 72), (64, 8192, 512), (2048, 1024, 192), (600, 288, 64), (200, 512, 1024),
                                       (4100, 2064, 128), (640, 8192, 128), (530, 8208, 192)])
def test_gemm_bf16_gated(m, inter, k):
    a = randn(m, k, dtype=torch.bfloat16, seed=15)
    gate, up = randn(inter, k, dtype=torch.bfloat16, seed=16, scale=0.3), randn(inter, k, dtype=torch.bfloat16, seed=17, scale=0.3)
    w = ops().interleave_gate_up(gate, up)
    out = torch.full((m, inter + 2), 3.0, dtype=torch.bfloat16, device=DEV)
    ops().gemm_bf16(a, w, out[:, :inter], gated=True)
    want = torch.nn.functional.silu(a.double() @ gate.double().T) * (a.double() @ up.double().T)
    assert rel(out[:, :inter], want) < 6e-3
    assert torch.all(out[:, inter:] == 3.0)


@pytest.mark.parametrize("m,n,k", [(4109, 4120, 192), (4096, 4096, 448)])
def test_gemm_bf16_ping_pong_with_whole_lines(m, n, k):
    """Outputs whose rows are 16-byte aligned leave the ping-pong kernel in whole cache lines: every epilogue, with edge tiles."""
    a, w = randn(m, k, dtype=torch.bfloat16, seed=25), randn(n, k, dtype=torch.bfloat16, seed=26, scale=0.3)
    want = a.double() @ w.double().T
    for out_dtype, accumulate in ((torch.float32, False), (torch.float32, True), (torch.bfloat16, False)):
        base = randn(m, n, seed=27).to(out_dtype)
        out = base.clone()
        ops().gemm_bf16(a, w, out, accumulate=accumulate)
        assert rel(out, want + (base.double() if accumulate else 0)) < (1e-5 if out_dtype == torch.float32 else 5e-3), (out_dtype, accumulate)
    gate, up = w[:n // 2 // 16 * 16], w[n // 2:n // 2 + n // 2 // 16 * 16]
    out = torch.full((m, gate.shape[0]), 3.0, dtype=torch.bfloat16, device=DEV)
    ops().gemm_bf16(a, ops().interleave_gate_up(gate.contiguous(), up.contiguous()), out, gated=True)
    assert rel(out, torch.nn.functional.silu(a.double() @ gate.double().T) * (a.double() @ up.double().T)) < 6e-3


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


@pytest.mark.parametrize("dim,dtype", [(2048, torch.bfloat16), (24, torch.bfloat16), (37, torch.bfloat16), (100, torch.float32)])
def test_embed_with_the_first_half_of_a_norm(dim, dtype):
    """The fetch of token rows that also writes them times a norm's weights in bfloat16 and their sums of squares (widths with and
    without the four-channel path), against the plain statement; with the product's share (times rsqrt(mean square + eps)) the
    rows are the norm's."""
    table = randn(50, dim, dtype=dtype, seed=10)
    toks = torch.tensor([3, 49, 0, 3, 17], dtype=torch.int32, device=DEV)
    g = (1 + 0.1 * randn(dim, seed=12)).contiguous()
    out, scaled, squares = torch.empty(5, dim, device=DEV), torch.empty(5, dim, dtype=torch.bfloat16, device=DEV), torch.empty(5, 1, device=DEV)
    ops().embed_handing(table, toks, out, g, scaled, squares)
    rows = table[toks.long()].double()
    assert torch.equal(out, rows.float())
    assert torch.equal(scaled, (g * out).to(torch.bfloat16))
    assert rel(squares[:, 0], (rows ** 2).sum(1)) < 1e-6
    normed = scaled.double() * torch.rsqrt(squares.double() / dim + 1e-5)
    assert rel(normed, g.double() * rows * torch.rsqrt((rows ** 2).mean(1, keepdim=True) + 1e-5)) < 5e-3


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


@pytest.mark.parametrize("m,d,k1,n2,gated", [(1, 2048, 2048, 3072, False), (8, 2048, 8192, 16384, True), (8, 2048, 2048, 16384, True), (9, 2048, 2048, 3072, False),
                                            (16, 136, 264, 96, False), (5, 3072, 3072, 5120, False), (3, 4096, 4096, 6144, False), (7, 264, 136, 64, True),
                                            (64, 2048, 8192, 16384, True), (64, 2048, 2048, 3072, False), (40, 2048, 8192, 3072, False), (17, 2048, 8192, 16384, True),
                                            (100, 4096, 14336, 6144, False), (128, 3072, 8192, 16384, True), (33, 1024, 512, 12288, False),
                                            (24, 2048, 2048, 16384, True), (24, 2048, 8192, 3072, False), (14, 2048, 2048, 16384, True), (32, 2048, 2048, 2048, False),
                                            (17, 264, 136, 12288, False), (13, 4096, 4096, 28672, True),
                                            # strips of 16 weight rows where strips of 8 would make more pieces than the reader takes (9 to 16 rows), and
                                            # from 4 rows on for the product that hands on with 256 strips or more
                                            (12, 3072, 8192, 5120, False), (16, 3072, 3072, 16384, True), (8, 4096, 14336, 6144, False), (4, 4096, 4096, 28672, True),
                                            # the rows of prompts: from the tiles of 128 x 128 (or the kernel that adds the shares of k) to the gated
                                            # product on the kernel with tiles of 256 x 256
                                            (2048, 2048, 2048, 16384, True), (2048, 2048, 8192, 16384, True), (1024, 2048, 2048, 16384, True),
                                            (1500, 3072, 1024, 16384, True),
                                            # ... with tiles of 256 x 256 for three quarters of the compute units
                                            (640, 2048, 2048, 16384, True), (530, 2048, 8192, 16384, True)])
def test_norm_handed_from_one_product_to_the_next(m, d, k1, n2, gated):
    """A product that adds onto rows x also writes g * x and the pieces of the rows' sums of squares; the next product reads
    g * x and multiplies its results by rsqrt(mean(x^2) + eps).  The rows x are what the plain product leaves, bit for bit; the
    second product's results are as near the 64-bit norm and product as those of the norm's own kernel followed by the product."""
    o = ops()
    eps = 1e-5
    a = randn(m, k1, dtype=torch.bfloat16, seed=1)
    w1 = randn(d, k1, dtype=torch.bfloat16, seed=2, scale=0.05)
    w2 = randn(n2, d, dtype=torch.bfloat16, seed=3, scale=0.05)
    g = (1 + 0.1 * randn(d, seed=4)).float()
    x0 = randn(m, d, seed=5)
    parts = o.gemm_bf16_norm_parts(m, d, k1)
    assert parts and o.gemm_bf16_takes_norm(m, n2, d, gated), "every case here is one the kernels take"
    plain_x = x0.clone()
    o.gemm_bf16(a, w1, plain_x, accumulate=True)
    x, scaled, squares = x0.clone(), torch.full((m, d), float("nan"), dtype=torch.bfloat16, device=DEV), torch.full((m, parts), float("nan"), device=DEV)
    o.gemm_bf16(a, w1, x, accumulate=True, norm_out=(g, scaled, squares))
    assert torch.equal(x, plain_x)
    assert torch.equal(scaled, (g * x).to(torch.bfloat16))
    assert rel(squares.double().sum(1), (x.double() ** 2).sum(1)) < 1e-6
    out_shape = (m, n2 // 2) if gated else (m, n2)
    out_dtype = torch.bfloat16 if gated else torch.float32
    w2k = o.interleave_gate_up(w2[:n2 // 2], w2[n2 // 2:]) if gated else w2
    handed = torch.empty(out_shape, dtype=out_dtype, device=DEV)
    o.gemm_bf16(scaled, w2k, handed, gated=gated, norm_in=(squares, eps))
    normed = torch.empty((m, d), dtype=torch.bfloat16, device=DEV)
    o.rmsnorm(x, g, eps, normed)
    usual = torch.empty(out_shape, dtype=out_dtype, device=DEV)
    o.gemm_bf16(normed, w2k, usual, gated=gated)
    xd = x.double()
    exact = (g.double() * xd * torch.rsqrt((xd ** 2).mean(1, keepdim=True) + eps)) @ w2.double().T
    if gated:
        exact = torch.nn.functional.silu(exact[:, :n2 // 2]) * exact[:, n2 // 2:]
    err_handed, err_usual = rel(handed, exact), rel(usual, exact)
    assert err_handed < 1.5 * err_usual + 1e-6, (err_handed, err_usual)


@pytest.mark.parametrize("m,d,k1", [(2048, 2048, 8192), (1100, 2048, 2048), (300, 2048, 2048), (2048, 3072, 8192), (700, 1024, 512), (130, 256, 192),
                                    (3000, 3072, 256), (4100, 2048, 256)])
def test_norm_handed_on_by_a_product_of_many_rows(m, d, k1):
    """The rows of prompts: the product that adds onto the residual writes g * x and the pieces of the rows' sums of squares from
    its tiles' epilogues (one piece per 128 columns), or from the kernel that adds the shares of k (one per 1024).  The rows are
    what the plain product leaves, bit for bit; sizes at which the kernels do not do it are refused."""
    o = ops()
    a = randn(m, k1, dtype=torch.bfloat16, seed=1)
    w1 = randn(d, k1, dtype=torch.bfloat16, seed=2, scale=0.05)
    g = (1 + 0.1 * randn(d, seed=4)).float()
    x0 = randn(m, d, seed=5)
    parts = o.gemm_bf16_norm_parts(m, d, k1)
    assert parts in (d // 128, d // 1024), parts
    plain_x = x0.clone()
    o.gemm_bf16(a, w1, plain_x, accumulate=True)
    x, scaled, squares = x0.clone(), torch.full((m, d), float("nan"), dtype=torch.bfloat16, device=DEV), torch.full((m, parts), float("nan"), device=DEV)
    o.gemm_bf16(a, w1, x, accumulate=True, norm_out=(g, scaled, squares))
    assert torch.equal(x, plain_x)
    assert torch.equal(scaled, (g * x).to(torch.bfloat16))
    assert rel(squares.double().sum(1), (x.double() ** 2).sum(1)) < 1e-6
    width = d // parts
    assert rel(squares.double(), (x.double() ** 2).view(m, parts, width).sum(2)) < 1e-6            # every piece is its columns' sum
    assert o.gemm_bf16_norm_parts(8192, 8192, 512) == 0 and o.gemm_bf16_norm_parts(300, 200, 512) == 0        # the ping-pong kernel; a ragged width
    with pytest.raises(o.KernelError):
        o.gemm_bf16(randn(8192, 512, dtype=torch.bfloat16, seed=1), randn(8192, 512, dtype=torch.bfloat16, seed=2), torch.zeros(8192, 8192, device=DEV),
                    accumulate=True, norm_out=((1 + 0 * randn(8192, seed=4)).float(), torch.empty(8192, 8192, dtype=torch.bfloat16, device=DEV), torch.empty(8192, 64, device=DEV)))


@pytest.mark.parametrize("m,hidden,n_heads,n_kv,hd,page_size,rotate,handed", [(64, 2048, 32, 8, 64, 16, True, True), (40, 2048, 32, 8, 64, 16, True, False),
                                                                              (128, 3072, 24, 8, 128, 16, True, True), (33, 512, 6, 1, 32, 8, False, False),
                                                                              (17, 4096, 32, 8, 128, 32, True, False), (100, 1024, 2, 1, 256, 16, True, True),
                                                                              # rows of prompts: tiles of 128 x 128 whose epilogue rotates and stores (two workgroups
                                                                              # of four waves a unit; one of eight), and shapes whose k is shared out over workgroups
                                                                              (2048, 2048, 32, 8, 64, 16, True, False), (1100, 256, 20, 2, 128, 16, True, True),
                                                                              (1100, 256, 80, 8, 32, 8, False, True), (300, 3072, 24, 8, 128, 16, True, True),
                                                                              (520, 512, 28, 2, 64, 16, True, False), (129, 2048, 32, 8, 64, 16, True, True)])
def test_qkv_product_that_rotates_and_fills_the_pages(m, hidden, n_heads, n_kv, hd, page_size, rotate, handed):
    """The q/k/v product whose last step rotates and writes the pages itself (the kernel that adds up the shares of k, or the
    epilogue over a tile of a prompt's rows) against the product followed by the kernel that does that, which
    `test_rope_store_writes_the_right_places` holds against the plain statement: the same queries and the same pages, also with
    a norm handed on."""
    o = ops()
    n = (n_heads + 2 * n_kv) * hd
    assert o.gemm_bf16_qkv_rope_store_takes(m, n, hidden, hd)
    a = randn(m, hidden, dtype=torch.bfloat16, seed=1)
    w = randn(n, hidden, dtype=torch.bfloat16, seed=2, scale=0.05)
    g = torch.Generator().manual_seed(9)
    ang = torch.rand(m, hd // 2, generator=g) * 6.28
    cos, sin = (torch.cos(ang).to(DEV), torch.sin(ang).to(DEV)) if rotate else (None, None)
    n_slots = 5
    pages_per = max(4, -(-2 * m // (n_slots * page_size)))
    n_pages = n_slots * pages_per + 2
    table = torch.randperm(n_pages, generator=g)[:n_slots * pages_per].view(n_slots, pages_per).to(torch.int32).to(DEV)
    slots = torch.randint(0, n_slots, (m,), generator=g).to(torch.int32)
    positions = torch.empty(m, dtype=torch.int32)
    seen = {}
    for i in range(m):                                                # distinct (slot, position) per row
        while True:
            p = int(torch.randint(0, pages_per * page_size, (1,), generator=g))
            if (int(slots[i]), p) not in seen:
                seen[(int(slots[i]), p)] = True
                positions[i] = p
                break
    slots, positions = slots.to(DEV), positions.to(DEV)
    norm_in = None
    fill = lambda: torch.full((n_pages, 2, n_kv, page_size, hd), 7.0, dtype=torch.bfloat16, device=DEV)
    want_cache, got_cache = fill(), fill()
    qkv = torch.empty(m, n, device=DEV)
    o.gemm_bf16(a, w, qkv)
    if handed:
        parts = min(16, o.gemm_bf16_qkv_rope_store_max_parts(m, n, hidden))
        squares = (torch.rand(m, parts, generator=g) * hidden / parts).to(DEV)
        norm_in = (squares, 1e-5)
        qkv *= torch.rsqrt(squares.sum(1, keepdim=True) / hidden + 1e-5)
    a_dim, kv_dim = n_heads * hd, n_kv * hd
    want_q = torch.empty(m, a_dim, dtype=torch.bfloat16, device=DEV)
    o.rope_store(qkv[:, :a_dim], qkv[:, a_dim:a_dim + kv_dim], qkv[:, a_dim + kv_dim:], cos, sin, positions, slots, table, want_q, want_cache, n_heads, n_kv, hd)
    got_q = torch.full((m, a_dim), float("nan"), dtype=torch.bfloat16, device=DEV)
    o.gemm_bf16_qkv_rope_store(a, w, cos, sin, positions, slots, table, got_q, got_cache, n_heads, n_kv, hd, norm_in)
    step = lambda t: t.float().abs().clamp_min(1e-3) * 2.0 ** -7          # a rounding step of bfloat16 at most: the two kernels may fuse a * cos - b * sin differently
    assert ((got_q.float() - want_q.float()).abs() <= step(want_q)).all()
    assert ((got_cache.float() - want_cache.float()).abs() <= step(want_cache)).all()
    assert float((got_q.float() != want_q.float()).float().mean()) < 0.01 and float((got_cache.float() != want_cache.float()).float().mean()) < 0.01


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


@pytest.mark.parametrize("vocab,light,heavy", [(100, 5, 40), (3000, 100, 1000), (3000, 17, 2999), (9000, 4000, 4095), (9000, 70, 5000)])
def test_a_draw_of_zero_takes_the_first_token_that_has_any_probability(vocab, light, heavy):
    """u = 0 stops at the first token whose probability is not zero (src/sampler/sampler.cpp:119-128), however little it weighs
    beside a later one: 1e-35 before a token of probability 1 is below the last bit of the running sum in 64-bit, so a thread that
    found where its tokens start by taking its own sum off the running one would start at 0 too and claim the draw."""
    from plain_sampler import sample
    logits = torch.full((3, vocab), -30.0)
    logits[:, heavy] = 0.0
    logits[0, light], logits[1, light], logits[2, light] = -0.8, -1.0, -1.04          # p = 1.8e-35, 3.8e-44 (subnormal), 0 at T = 0.01
    out = torch.empty(3, dtype=torch.int32, device=DEV)
    ops().sample_temperature(logits.to(DEV), torch.full((3,), 0.01, device=DEV), torch.zeros(3, device=DEV), out)
    assert [sample(row.numpy(), 0.01, 0, 1.0, 0.0) for row in logits] == [light, light, heavy]
    assert out.tolist() == [light, light, heavy]


def on_an_edge(logits, temperature, top_k, top_p, u, got, want):
    """Whether the plain sampler could give `got` for `want` by rounding alone: two tokens whose probabilities differ in the
    last bits change places in the order, or u, or top_p times the kept mass, falls within 2e-6 of a boundary."""
    from plain_sampler import sample
    p = torch.softmax(torch.from_numpy(logits).double() / temperature, 0)
    if abs(float(p[got]) - float(p[want])) <= 1e-6 * float(p[want]):
        return True
    near = set()
    for dp in (-2e-6, 0.0, 2e-6):
        for du in (-2e-6, 0.0, 2e-6):
            near.add(sample(logits, temperature, top_k, top_p if top_p >= 1.0 else min(max(top_p + dp, 1e-6), 1.0 - 1e-7),
                            min(max(u + du, 0.0), 1.0 - 2.0 ** -24)))
    return got in near


def filtered_on_device(logits, temps, ks, ps, us):
    n = logits.shape[0]
    out = torch.empty(n, dtype=torch.int32, device=DEV)
    ops().sample_filtered(logits.to(DEV), torch.tensor(temps, dtype=torch.float32, device=DEV), torch.tensor(ks, dtype=torch.int32, device=DEV),
                          torch.tensor(ps, dtype=torch.float32, device=DEV), torch.tensor(us, dtype=torch.float32, device=DEV), out)
    return out.tolist()


def test_filters_on_the_device_keep_what_they_should():
    """The sets that the filters leave, as the reference's test states them (tests/verify_sampler.py:161-166): among equal
    probabilities the lowest indices stay."""
    g = torch.Generator().manual_seed(3)
    us = torch.rand(300, generator=g).tolist()
    flat = torch.zeros(300, 10)
    assert set(filtered_on_device(flat, [1.0] * 300, [3] * 300, [1.0] * 300, us)) == {0, 1, 2}
    assert set(filtered_on_device(flat, [1.0] * 300, [0] * 300, [0.35] * 300, us)) == {0, 1, 2, 3}
    assert set(filtered_on_device(flat, [1.0] * 300, [7] * 300, [0.35] * 300, us)) == {0, 1, 2}          # 0.35 of the mass of seven
    peaked = torch.zeros(300, 20)
    peaked[:, 13] = 30.0
    assert set(filtered_on_device(peaked, [1.0] * 300, [0] * 300, [0.9] * 300, us)) == {13}
    assert set(filtered_on_device(peaked, [1.0] * 300, [1] * 300, [1.0] * 300, us)) == {13}
    wide = torch.zeros(300, 5000)                                   # equal probabilities far beyond one wave's reach
    wide[:, 4000:] = 1.0
    got = filtered_on_device(wide, [1.0] * 300, [600] * 300, [1.0] * 300, us)
    assert min(got) >= 4000 and max(got) < 4600 and len(set(got)) > 150
    got = filtered_on_device(wide, [1.0] * 300, [1300] * 300, [1.0] * 300, us)                            # all of the likely ones and 300 of the rest
    assert set(t for t in got if t < 4000) <= set(range(300)) and any(t < 4000 for t in got) and max(got) < 5000


def test_sample_filtered_matches_the_plain_sampler():
    """Top-k and top-p on the device against the plain sampler, row by row: random logits, logits on a coarse grid (many
    tokens of exactly equal probability, so that the filters cut through groups of equals), and the real vocabulary."""
    from plain_sampler import sample
    g = torch.Generator().manual_seed(1)
    settings = [(1.0, 0, 0.9), (0.8, 0, 0.5), (1.0, 0, 0.05), (1.0, 3, 1.0), (1.5, 50, 1.0), (1.0, 5, 0.9), (0.7, 1, 1.0), (1.0, 4, 0.3),
                (0.3, 0, 0.999), (2.0, 40, 0.95), (1.0, 10 ** 6, 0.7), (1.0, 0, 2.0 ** -20)]
    exact = total = 0
    for vocab, coarse in ((2, False), (5, False), (100, False), (100, True), (3001, False), (3001, True), (128256, False), (128256, True)):
        rows = []
        for t, k, p in settings:
            if not (0 < k < vocab or p < 1.0):
                continue
            for u in torch.rand(2 if vocab > 100000 else 6, generator=g).tolist() + [0.0, 1.0 - 2.0 ** -24]:
                rows.append((t, k, p, u))
        logits = 2 * torch.randn(len(rows), vocab, generator=g)
        if coarse:
            logits = torch.round(logits * 2) / 2
        got = filtered_on_device(logits, *zip(*rows))
        for i, (t, k, p, u) in enumerate(rows):
            row = logits[i].numpy()
            want = sample(row, t, k, p, np.float32(u))
            total += 1
            exact += got[i] == want
            assert got[i] == want or on_an_edge(row, t, k, p, u, got[i], want), (vocab, coarse, i, (t, k, p, u), got[i], want)
    assert exact >= 0.98 * total, (exact, total)


def test_rows_of_every_kind_of_sampler_in_one_call():
    """Greedy, plain and filtered samplers side by side get what each gets alone, and every one draws from its own stream."""
    from geneinfer_amd.sampling import Sampler, SamplerConfig, sample_rows
    g = torch.Generator().manual_seed(5)
    vocab = 777
    configs = [SamplerConfig(0.0), SamplerConfig(0.9, seed=4), SamplerConfig(1.0, top_k=7, seed=5), SamplerConfig(0.0), SamplerConfig(0.7, top_p=0.8, seed=6),
               SamplerConfig(1.2, seed=7), SamplerConfig(1.0, top_k=20, top_p=0.5, seed=8)]
    together = [Sampler(c, vocab) for c in configs]
    alone = [Sampler(c, vocab) for c in configs]
    for step in range(5):
        logits = (2 * torch.randn(len(configs), vocab, generator=g)).to(DEV)
        got = sample_rows(logits, together)
        want = [sample_rows(logits[i:i + 1], [alone[i]])[0] for i in range(len(configs))]
        assert got == want, (step, got, want)
        assert [s.stream.state for s in together] == [s.stream.state for s in alone]
    some = [together[i] for i in (2, 4, 6)]                           # only filtered ones: no gathering
    logits = (2 * torch.randn(3, vocab, generator=g)).to(DEV)
    assert sample_rows(logits, some) == [sample_rows(logits[i:i + 1], [alone[j]])[0] for i, j in enumerate((2, 4, 6))]


# ------------------------------------------------------------------------------------- attention
def build_paged(requests, n_kv, hd, page_size, dtype, seed, scale_one=None, gone_before=None, shape_keys=None):
    """Dense keys/values per request, written into a paged cache with scrambled pages and a rim of
    NaN pages that nothing may touch.  requests: list of context lengths.  gone_before: per request index, a position;
    pages that lie wholly before it have been given back (a window has passed them): their table entries are -1 and
    nothing of them is in the cache.  Returns cache, table, dense."""
    g = torch.Generator().manual_seed(seed)
    n_pages_needed = sum(-(-n // page_size) for n in requests)
    n_pages = n_pages_needed + 3
    perm = torch.randperm(n_pages, generator=g).tolist()
    cache = torch.full((n_pages, 2, n_kv, page_size, hd), float("nan"), dtype=dtype)
    width = max(-(-n // page_size) for n in requests) + 2
    table = torch.full((len(requests) + 1, width), -1, dtype=torch.int32)
    dense, nxt = [], 0
    for slot, n in enumerate(requests):
        k = torch.randn(n, n_kv, hd, generator=g).to(dtype)
        v = torch.randn(n, n_kv, hd, generator=g).to(dtype)
        if scale_one is not None and n > scale_one[0]:
            k[scale_one[0]] *= scale_one[1]                    # one far key that must stand out
        if shape_keys is not None:
            k = shape_keys(slot, k.float()).to(dtype)
        dense.append((k, v))
        for i in range(-(-n // page_size)):
            if gone_before is not None and (i + 1) * page_size <= gone_before.get(slot, 0):
                continue
            page = perm[nxt]; nxt += 1
            table[slot + 1, i] = page                          # slot 0 of the table stays unused (-1)
            cache[page] = 0
            m = min(page_size, n - i * page_size)
            cache[page, 0, :, :m, :] = k[i * page_size:i * page_size + m].permute(1, 0, 2)
            cache[page, 1].view(n_kv, hd, page_size)[:, :, :m] = v[i * page_size:i * page_size + m].permute(1, 2, 0)
    return cache.to(DEV), table.to(DEV), dense


def plain_attention_rows(q, dense, rows, n_heads, n_kv, hd, window):
    """rows: (slot, pos) per row of q [n, heads*hd]; float64 softmax(q k / sqrt(hd)) v over keys <= pos."""
    out = torch.zeros(q.shape[0], n_heads, hd, dtype=torch.float64)
    qd = q.double().cpu().view(-1, n_heads, hd)
    for i, (slot, pos) in enumerate(rows):
        k, v = dense[slot]
        lo = max(0, pos - window + 1) if window else 0
        for h in range(n_heads):
            kv = h // (n_heads // n_kv)
            s = (k[lo:pos + 1, kv].double() @ qd[i, h]) / math.sqrt(hd)
            out[i, h] = torch.softmax(s, 0) @ v[lo:pos + 1, kv].double()
    return out.view(q.shape[0], n_heads * hd)


ATT_CASES = [  # n_heads, n_kv, hd, page_size, window
    (4, 2, 64, 16, None), (3, 1, 32, 16, None), (8, 8, 128, 32, None), (6, 2, 96, 16, None), (4, 4, 64, 16, 40), (32, 8, 64, 16, None),
    (5, 5, 48, 16, None), (2, 1, 16, 4, 9), (4, 2, 256, 16, None), (8, 2, 128, 16, 50), (6, 3, 128, 48, None),
]


SEGMENTS = {
    # request 0: rows at positions 150..299 (a portion on top of 150 cached positions); request 1: its last row;
    # request 2: its only row; request 3: rows 0..76 (a whole prompt); request 4: its last row
    "long portions": [(0, 150, 150), (1, 130, 1), (2, 0, 1), (3, 0, 77), (4, 529, 1)],
    # short portions, 60 rows in all: the matrix-core path takes them row by row through the decode kernel
    "short portions": [(0, 250, 50), (1, 130, 1), (2, 0, 1), (3, 70, 7), (4, 527, 3)],
    # short portions that sum to more than 64 rows stay tiles
    "many short portions": [(0, 240, 60), (1, 130, 1), (3, 47, 30), (4, 490, 40)],
    # portions of several tiles: a late tile shares its workgroup with an early one (3 tiles: the middle one alone; 4: two pairs)
    "several tiles": [(0, 0, 300), (1, 130, 1), (4, 100, 430)],
}


@pytest.mark.parametrize("n_heads,n_kv,hd,ps,window", ATT_CASES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("portions,tile", [(name, 0) for name in SEGMENTS] + [("long portions", 128), ("several tiles", 128)])
def test_attention_over_pages(n_heads, n_kv, hd, ps, window, dtype, portions, tile, monkeypatch):
    """Portions of prompts on top of an existing cache, beside single decoded rows, on scrambled pages.
    tile: rows of a prompt tile (0: as the step's size decides, which is 64 for steps as small as these)."""
    from geneinfer_amd.parts import StepContext
    monkeypatch.setattr(ops().AttentionPlan, "TILE", tile)
    contexts = [300, 131, 1, 77, 530]
    segs = SEGMENTS[portions]
    # with a window, the pages that no row of the step can see have been given back
    gone = {slot: max(0, pos0 - window + 1) for slot, pos0, _ in segs} if window else None
    cache, table, dense = build_paged(contexts, n_kv, hd, ps, dtype, seed=hd + n_heads, gone_before=gone)
    if window:
        assert int((table[1:] == -1).sum()) > int((build_paged(contexts, n_kv, hd, ps, dtype, seed=hd + n_heads)[1][1:] == -1).sum())
    rows, seg_start, seg_len, seg_pos0, seg_slot = [], [], [], [], []
    for slot, pos0, n in segs:
        seg_start.append(len(rows)); seg_len.append(n); seg_pos0.append(pos0); seg_slot.append(slot + 1)
        rows += [(slot, pos0 + i) for i in range(n)]
    T = len(rows)
    q = randn(T, n_heads * hd, dtype=dtype, seed=3)
    pos = torch.tensor([p for _, p in rows], dtype=torch.int32, device=DEV)
    slots = torch.tensor([s + 1 for s, _ in rows], dtype=torch.int32, device=DEV)
    ctx = StepContext(n_rows=T, dtype=dtype, device=torch.device(DEV), tokens=pos, row_pos=pos, row_slot=slots, seg_slot=seg_slot,
                      seg_start=seg_start, seg_len=seg_len, seg_pos0=seg_pos0)
    out = torch.full((T, n_heads * hd), float("nan"), dtype=dtype, device=DEV)
    before = cache.clone()
    ops().attention(q, cache, out, ctx, table, n_heads, n_kv, hd, window)
    want = plain_attention_rows(q, dense, rows, n_heads, n_kv, hd, window)
    err = rel(out, want)
    assert err < (2e-6 if dtype == torch.float32 else 8e-3), err
    assert torch.equal(torch.nan_to_num(cache, nan=-1.0), torch.nan_to_num(before, nan=-1.0)), "attention wrote into the cache"


@pytest.mark.parametrize("n_heads,n_kv,hd,ps,window", [(4, 2, 64, 16, None), (3, 1, 32, 16, None), (8, 8, 128, 32, None), (6, 2, 96, 16, 700), (4, 4, 64, 16, 450),
                                                       (4, 1, 128, 16, 600)])
def test_few_prompt_tiles_over_a_long_context_share_their_keys_out(n_heads, n_kv, hd, ps, window):
    """Two portions on top of long cached contexts: few tiles, so each tile's keys go to several workgroups and a combine
    kernel; among the keys one far one is scaled so that a lost share would show."""
    from geneinfer_amd.parts import StepContext
    o = ops()
    contexts = [1500, 730, 40]
    segs = [(0, 1400, 100), (1, 600, 130), (2, 39, 1)]
    gone = {slot: max(0, pos0 - window + 1) for slot, pos0, _ in segs} if window else None          # what a window has given back
    cache, table, dense = build_paged(contexts, n_kv, hd, ps, torch.bfloat16, seed=hd + n_heads + 7, scale_one=(333, 3.0), gone_before=gone)
    rows, seg_start, seg_len, seg_pos0, seg_slot = [], [], [], [], []
    for slot, pos0, n in segs:
        seg_start.append(len(rows)); seg_len.append(n); seg_pos0.append(pos0); seg_slot.append(slot + 1)
        rows += [(slot, pos0 + i) for i in range(n)]
    T = len(rows)
    q = randn(T, n_heads * hd, dtype=torch.bfloat16, seed=3)
    pos = torch.tensor([p for _, p in rows], dtype=torch.int32, device=DEV)
    slots = torch.tensor([s_ + 1 for s_, _ in rows], dtype=torch.int32, device=DEV)
    ctx = StepContext(n_rows=T, dtype=torch.bfloat16, device=torch.device(DEV), tokens=pos, row_pos=pos, row_slot=slots, seg_slot=seg_slot,
                      seg_start=seg_start, seg_len=seg_len, seg_pos0=seg_pos0)
    assert o.prompt_attention_splits(3, n_heads, 1500 if not window else window + 128) > 1
    out = torch.full((T, n_heads * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    o.attention(q, cache, out, ctx, table, n_heads, n_kv, hd, window)
    want = plain_attention_rows(q, dense, rows, n_heads, n_kv, hd, window)
    assert rel(out, want) < 8e-3, rel(out, want)


@pytest.mark.parametrize("window", [None, 200])
def test_many_prompt_tiles_of_many_heads(window):
    """More workgroups than compute units at head size 64 (5 pairs of tiles x 64 heads): the step takes the kernel with a
    workgroup per tile, several to a compute unit, which head size 128 always takes.  A whole prompt of 900 rows, a portion of
    130 rows on 300 cached positions and a single row; with a window the pages behind it are gone."""
    from geneinfer_amd.parts import StepContext
    n_heads, n_kv, hd, ps = 64, 16, 64, 16
    contexts = [900, 430, 50]
    segs = [(0, 0, 900), (1, 300, 130), (2, 49, 1)]
    gone = {slot: max(0, pos0 - window + 1) for slot, pos0, _ in segs} if window else None
    cache, table, dense = build_paged(contexts, n_kv, hd, ps, torch.bfloat16, seed=5, scale_one=(77, 3.0), gone_before=gone)
    rows, seg_start, seg_len, seg_pos0, seg_slot = [], [], [], [], []
    for slot, pos0, n in segs:
        seg_start.append(len(rows)); seg_len.append(n); seg_pos0.append(pos0); seg_slot.append(slot + 1)
        rows += [(slot, pos0 + i) for i in range(n)]
    T = len(rows)
    q = randn(T, n_heads * hd, dtype=torch.bfloat16, seed=3)
    pos = torch.tensor([p for _, p in rows], dtype=torch.int32, device=DEV)
    slots = torch.tensor([s_ + 1 for s_, _ in rows], dtype=torch.int32, device=DEV)
    ctx = StepContext(n_rows=T, dtype=torch.bfloat16, device=torch.device(DEV), tokens=pos, row_pos=pos, row_slot=slots, seg_slot=seg_slot,
                      seg_start=seg_start, seg_len=seg_len, seg_pos0=seg_pos0)
    plan = ops().AttentionPlan(seg_start, seg_len, seg_pos0, seg_slot, DEV)
    assert plan.paired and plan.tile == 128 and plan.n_tiles // 2 * n_heads > 256
    out = torch.full((T, n_heads * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops().attention(q, cache, out, ctx, table, n_heads, n_kv, hd, window)
    want = plain_attention_rows(q, dense, rows, n_heads, n_kv, hd, window)
    assert rel(out, want) < 8e-3, rel(out, want)


@pytest.mark.parametrize("n_heads,n_kv,hd", [(4, 2, 64), (4, 2, 128), (64, 16, 64)])
def test_prompt_attention_with_scores_that_climb_along_the_context(n_heads, n_kv, hd):
    """Every query points along one direction and the keys' share of that direction climbs with their position, by 2 to 12
    units of log2 e from one tile of 64 keys to the next, and falls again behind position 800: the running maximum of a
    row moves in every tile, by less and by more than what the kernels let it lag behind.  Scores reach 60 and more, so a
    maximum applied wrongly once is a factor and not a rounding error.  A whole prompt of several tiles, a portion on a
    cached context and a single row (in the last case: more workgroups than compute units, the other prompt kernel)."""
    from geneinfer_amd.parts import StepContext
    ps = 16
    contexts = [1200, 900, 50]
    segs = [(0, 0, 1200), (1, 700, 200), (2, 49, 1)]
    g = torch.Generator().manual_seed(11)
    direction = torch.nn.functional.normalize(torch.randn(n_kv, hd, generator=g), dim=-1)
    pos_all = torch.arange(1200, dtype=torch.float32)
    # slope per position in nats of the final score: gentle, then steep, then falling
    slope = torch.where(pos_all < 300, 0.02, torch.where(pos_all < 800, 0.13, -0.09))
    height = torch.cumsum(slope, 0)                                        # the score a unit query gives the key at a position
    q_gain = 3.0

    def shape_keys(slot, k):
        n = k.shape[0]
        return 0.3 * k + (height[:n] * math.sqrt(hd) / q_gain)[:, None, None] * direction[None]

    cache, table, dense = build_paged(contexts, n_kv, hd, ps, torch.bfloat16, seed=hd + 2, shape_keys=shape_keys)
    rows, seg_start, seg_len, seg_pos0, seg_slot = [], [], [], [], []
    for slot, pos0, n in segs:
        seg_start.append(len(rows)); seg_len.append(n); seg_pos0.append(pos0); seg_slot.append(slot + 1)
        rows += [(slot, pos0 + i) for i in range(n)]
    T = len(rows)
    q = (q_gain * direction.repeat_interleave(n_heads // n_kv, 0).reshape(1, n_heads * hd) + 0.3 * torch.randn(T, n_heads * hd, generator=g)).to(torch.bfloat16).to(DEV)
    pos = torch.tensor([p for _, p in rows], dtype=torch.int32, device=DEV)
    slots = torch.tensor([s_ + 1 for s_, _ in rows], dtype=torch.int32, device=DEV)
    ctx = StepContext(n_rows=T, dtype=torch.bfloat16, device=torch.device(DEV), tokens=pos, row_pos=pos, row_slot=slots, seg_slot=seg_slot,
                      seg_start=seg_start, seg_len=seg_len, seg_pos0=seg_pos0)
    out = torch.full((T, n_heads * hd), float("nan"), dtype=torch.bfloat16, device=DEV)
    ops().attention(q, cache, out, ctx, table, n_heads, n_kv, hd, None)
    k0 = dense[0][0]
    top = float((k0[:, 0].double() @ q[0].double().cpu().view(n_heads, hd)[0]).max() / math.sqrt(hd))
    assert top > 40, top                                                   # the scores do climb as meant
    want = plain_attention_rows(q, dense, rows, n_heads, n_kv, hd, None)
    assert rel(out, want) < 8e-3, rel(out, want)
    worst_row = float(((out.double().cpu() - want).norm(dim=1) / want.norm(dim=1)).max())
    assert worst_row < 3e-2, worst_row                                     # no row is off by a factor


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_finds_one_far_key(dtype):
    """Among 700 keys one is scaled so that its score stands out: the output must be its value."""
    from geneinfer_amd.parts import StepContext
    n_heads, n_kv, hd, ps = 4, 2, 64, 16
    cache, table, dense = build_paged([700], n_kv, hd, ps, dtype, seed=1)
    k, v = dense[0]
    target = 37
    q = (k[target].float().repeat_interleave(n_heads // n_kv, 0) * 3.0).reshape(1, n_heads * hd).to(dtype).to(DEV)
    pos = torch.tensor([699], dtype=torch.int32, device=DEV)
    slots = torch.tensor([1], dtype=torch.int32, device=DEV)
    ctx = StepContext(n_rows=1, dtype=dtype, device=torch.device(DEV), tokens=pos, row_pos=pos, row_slot=slots, seg_slot=[1], seg_start=[0],
                      seg_len=[1], seg_pos0=[699])
    out = torch.empty(1, n_heads * hd, dtype=dtype, device=DEV)
    ops().attention(q, cache, out, ctx, table, n_heads, n_kv, hd, None)
    want = plain_attention_rows(q, dense, [(0, 699)], n_heads, n_kv, hd, None)
    assert rel(out, want) < (2e-6 if dtype == torch.float32 else 8e-3)
    assert rel(out.view(n_heads, hd)[0], v[target, 0]) < 2e-2          # the softmax is nearly one-hot on the target


@pytest.mark.parametrize("n_heads,n_kv,hd,ps,window", ATT_CASES)
@pytest.mark.parametrize("target_waves", [4096, 64])
def test_decode_attention_from_unrotated_products(n_heads, n_kv, hd, ps, window, target_waves, monkeypatch):
    """Single decoded rows whose keys and values are not in the cache yet: one kernel rotates q and k,
    attends (its own position included) and writes k and v to the right places, in one split and in several."""
    from geneinfer_amd.parts import StepContext
    shape = ops().decode_attention_shape
    monkeypatch.setattr(ops(), "decode_attention_shape", lambda *a, **k: shape(*a[:5], target_waves=target_waves))
    contexts = [300, 131, 1, 77, 530, 16, 17, 1200, 32, 33]           # the new row's position is the last of each
    gone = {slot: max(0, n - window) for slot, n in enumerate(contexts)} if window else None        # what a window has given back
    cache, table, dense = build_paged(contexts, n_kv, hd, ps, torch.bfloat16, seed=hd + n_heads + 1, gone_before=gone)
    T = len(contexts)
    pos = torch.tensor([n - 1 for n in contexts], dtype=torch.int32, device=DEV)
    slots = torch.arange(1, T + 1, dtype=torch.int32, device=DEV)
    a, kvd = n_heads * hd, n_kv * hd
    qkv = randn(T, a + 2 * kvd, seed=31)
    inv = torch.tensor([1.0 / (10000.0 ** (2 * k / hd)) for k in range(hd // 2)], dtype=torch.float64, device=DEV)
    cos, sin = torch.empty(T, hd // 2, device=DEV), torch.empty(T, hd // 2, device=DEV)
    ops().rope_cos_sin(pos, inv, cos, sin)

    def rotated(x, heads):
        x = x.double().cpu().view(T, heads, hd)
        c, s_ = torch.cat([cos, cos], -1).double().cpu()[:, None, :], torch.cat([sin, sin], -1).double().cpu()[:, None, :]
        return x * c + torch.cat([-x[..., hd // 2:], x[..., :hd // 2]], -1) * s_

    q_rot = rotated(qkv[:, :a], n_heads).to(torch.bfloat16).view(T, a)
    k_rot = rotated(qkv[:, a:a + kvd], n_kv).to(torch.bfloat16)
    v_new = qkv[:, a + kvd:].cpu().view(T, n_kv, hd).to(torch.bfloat16)
    want_cache = cache.clone()
    for i, n in enumerate(contexts):                                   # the row's own place: empty before, k and v after
        dense[i][0][n - 1], dense[i][1][n - 1] = k_rot[i], v_new[i]
        page, place = int(table[i + 1, (n - 1) // ps]), (n - 1) % ps
        cache[page, 0, :, place, :] = 0
        cache[page, 1].view(n_kv, hd, ps)[:, :, place] = 0
        want_cache[page, 0, :, place, :] = k_rot[i].to(DEV)
        want_cache[page, 1].view(n_kv, hd, ps)[:, :, place] = v_new[i].to(DEV)
    ctx = StepContext(n_rows=T, dtype=torch.bfloat16, device=torch.device(DEV), tokens=pos, row_pos=pos, row_slot=slots,
                      seg_slot=list(range(1, T + 1)), seg_start=list(range(T)), seg_len=[1] * T, seg_pos0=[n - 1 for n in contexts])
    out = torch.full((T, a), float("nan"), dtype=torch.bfloat16, device=DEV)
    done = ops().attention_from_products(qkv[:, :a], qkv[:, a:a + kvd], qkv[:, a + kvd:], cos, sin, cache, out, ctx, table, n_heads, n_kv, hd, window)
    if not ops().attention_bf16_supports(hd, ps, False):
        assert done is False and bool(torch.isnan(out.float()).all())    # refused: the caller rotates and stores first
        return
    assert done is True
    want = plain_attention_rows(q_rot, dense, [(i, n - 1) for i, n in enumerate(contexts)], n_heads, n_kv, hd, window)
    assert rel(out, want) < 8e-3, rel(out, want)
    got_c, want_c = torch.nan_to_num(cache.float(), nan=-1.0), torch.nan_to_num(want_cache.float(), nan=-1.0)
    assert rel(got_c, want_c) < 1e-3                                  # a rotated key may round the other way in 32-bit
    assert float(((got_c - want_c).abs() > 0.02 * want_c.abs() + 1e-6).sum()) == 0
    # read-only use of another layer's pages (which now hold the rows' keys and values): the same output, the cache untouched
    out2, before = torch.full_like(out, float("nan")), cache.clone()
    assert ops().attention_from_products(qkv[:, :a], None, None, cos, sin, cache, out2, ctx, table, n_heads, n_kv, hd, window)
    assert rel(out2, want) < 8e-3
    assert torch.equal(torch.nan_to_num(cache, nan=-1.0), torch.nan_to_num(before, nan=-1.0))


@pytest.mark.parametrize("hd", [64, 128])
def test_decode_attention_shape_leaves_no_nearly_empty_round(hd):
    """The cut of the context over workgroups: whatever the number of rows, the context is either not cut at all (a workgroup of 4
    or 8 waves per row and group of heads, where the busiest compute unit is expected to be done no later than the chip's memory
    plus a merging kernel), or the workgroups fit the chip at once, or their last round is not a small remainder; pieces never
    fall under 64 positions and the waves cover the span."""
    o = ops()
    n_heads, n_kv, span = 32, 8, 4096
    uncut = 0
    for rows in list(range(17, 130)) + [192, 256, 500]:
        splits, n_waves = o.decode_attention_shape(rows, n_heads, n_kv, hd, span)
        assert 1 <= n_waves <= 8 and splits >= 1 and not 5 <= n_waves <= 7
        single = o._decode_single_split(rows * n_kv, span, hd, 8)
        if single is not None:
            assert (splits, n_waves) == single and splits == 1 and n_waves in (4, 8)
            uncut += 1
            continue
        assert splits * n_waves == 1 or o._decode_piece(span, splits * n_waves) >= 64
        rounds = rows * n_kv * splits / o._decode_places(hd, False, n_waves, 4)
        plain = o._decode_plain_shape(rows * n_kv, span, 8)
        if (splits, n_waves) != plain:
            assert rounds <= 1, (rows, splits, n_waves, rounds)
        else:
            assert rounds <= 1 or rounds - int(rounds) == 0 or rounds - int(rounds) >= 0.3, (rows, splits, n_waves, rounds)
    assert 30 <= uncut <= 100                              # (a workgroup for every compute unit, or a whole number of them: 32, 64, 96, 128 rows; not 40 or 65)
    assert o._decode_single_split(64 * n_kv, span, hd, 8) is not None and o._decode_single_split(65 * n_kv, span, hd, 8) is None
    assert o._decode_single_split(8 * n_kv, span, hd, 8) is None
    for rows in range(1, 17):                              # the kernel that also rotates and stores: the plain rule at 64 channels, one round at 128
        splits, n_waves = o.decode_attention_shape(rows, n_heads, n_kv, hd, span, fused=True)
        if hd == 64:
            assert (splits, n_waves) == o._decode_plain_shape(rows * n_kv, span, 8, small=True)
            assert o._decode_piece(span, splits * n_waves) >= 32 and (n_waves == 8) == (rows * n_kv <= 64 or splits == 1)
        else:
            assert rows * n_kv * splits <= o._decode_places(hd, True, n_waves, 4) or (splits, n_waves) == o._decode_plain_shape(rows * n_kv, span, 8)
            assert o._decode_piece(span, splits * n_waves) >= 64


def test_rope_store_writes_the_right_places():
    n_heads, n_kv, hd, ps = 4, 2, 32, 16
    n_pages = 5
    cache = torch.full((n_pages, 2, n_kv, ps, hd), -777.25, device=DEV)
    table = torch.tensor([[-1, -1, -1], [3, 0, 4]], dtype=torch.int32, device=DEV)
    T = 3
    pos = torch.tensor([15, 16, 17], dtype=torch.int32, device=DEV)     # the last place of a page, then the next page
    slots = torch.ones(T, dtype=torch.int32, device=DEV)
    qkv = randn(T, (n_heads + 2 * n_kv) * hd, seed=20)
    a, kvd = n_heads * hd, n_kv * hd
    inv = torch.tensor([1.0 / (10000.0 ** (2 * k / hd)) for k in range(hd // 2)], dtype=torch.float64, device=DEV)
    cos, sin = torch.empty(T, hd // 2, device=DEV), torch.empty(T, hd // 2, device=DEV)
    ops().rope_cos_sin(pos, inv, cos, sin)
    q_out = torch.empty(T, a, device=DEV)
    ops().rope_store(qkv[:, :a], qkv[:, a:a + kvd], qkv[:, a + kvd:], cos, sin, pos, slots, table, q_out, cache, n_heads, n_kv, hd)

    def rotate_half_form(x, heads):          # x*cos + rotate_half(x)*sin with cos/sin doubled over both halves (tests/verify_kernels.py:284-291)
        x = x.double().cpu().view(T, heads, hd)
        ang = pos.double().cpu()[:, None] * inv.cpu()[None, :]
        c, s_ = torch.cat([ang.cos(), ang.cos()], -1)[:, None, :], torch.cat([ang.sin(), ang.sin()], -1)[:, None, :]
        rot = torch.cat([-x[..., hd // 2:], x[..., :hd // 2]], -1)
        return x * c + rot * s_

    assert rel(q_out.view(T, n_heads, hd), rotate_half_form(qkv[:, :a], n_heads)) < 2e-6
    k_want = rotate_half_form(qkv[:, a:a + kvd], n_kv)
    v_want = qkv[:, a + kvd:].double().cpu().view(T, n_kv, hd)
    for t, (page, place) in enumerate([(3, 15), (0, 0), (0, 1)]):
        assert rel(cache[page, 0, :, place, :], k_want[t]) < 2e-6
        assert rel(cache[page, 1].view(n_kv, hd, ps)[:, :, place], v_want[t]) < 1e-7
    touched = torch.zeros_like(cache, dtype=torch.bool)
    for page, place in [(3, 15), (0, 0), (0, 1)]:
        touched[page, 0, :, place, :] = True
        touched[page, 1].view(n_kv, hd, ps)[:, :, place] = True
    assert torch.all(cache[~touched] == -777.25), "rope_store wrote outside its places"
