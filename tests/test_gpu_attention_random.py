"""Steps drawn at random through the bfloat16 attention kernels (both prompt kernels, the decode kernel, the combine of shared-out
keys) against a dense 64-bit computation: one to four requests that bring a single row, a short portion or up to 1,400 rows, on top
of up to 3,000 cached positions, head sizes 64 and 128 with one to five query heads per key/value head, pages of 16 to 64 positions on
scrambled page numbers between pages of NaN, with and without a window whose passed pages are gone from the table."""
import random

import pytest
import torch

pytestmark = pytest.mark.gpu
dev = "cuda:0"


def dense_ref(q, K, V, rows, H, KV, hd, window):
    out = torch.zeros(len(rows), H * hd, dtype=torch.float64, device=dev)
    grp = H // KV
    # batch per request
    byreq = {}
    for i, (s, p) in enumerate(rows): byreq.setdefault(s, []).append((i, p))
    for s, lst in byreq.items():
        idx = torch.tensor([i for i, _ in lst], device=dev); pos = torch.tensor([p for _, p in lst], device=dev)
        L = int(pos.max()) + 1
        k = K[s][:L].double(); v = V[s][:L].double()                 # [L, KV, hd]
        qq = q[idx].double().view(-1, H, hd)
        kk = k.repeat_interleave(grp, dim=1); vv = v.repeat_interleave(grp, dim=1)
        sc = torch.einsum("thd,lhd->thl", qq, kk) * hd ** -0.5
        ar = torch.arange(L, device=dev)[None, None, :]
        mask = ar <= pos[:, None, None]
        if window: mask = mask & (ar > pos[:, None, None] - window)
        sc = sc.masked_fill(~mask, float("-inf"))
        o = torch.einsum("thl,lhd->thd", torch.softmax(sc, dim=-1), vv)
        out[idx] = o.reshape(-1, H * hd)
    return out


@pytest.mark.parametrize("case", range(40))
def test_a_step_drawn_at_random(case):
    from geneinfer_amd.kernels import ops
    from geneinfer_amd.parts import StepContext
    rng = random.Random(100 + case)
    torch.manual_seed(case)
    hd = rng.choice([64, 128, 128]); KV = rng.choice([1, 2, 4, 8]); H = KV * rng.choice([1, 2, 4, 5]); page = rng.choice([16, 16, 32, 48, 64])
    window = rng.choice([None, None, rng.randrange(20, 700)])
    R = rng.randrange(1, 5)
    segs = []
    for s in range(R):
        kind = rng.random()
        start = rng.choice([0, 0, rng.randrange(1, 3000)])
        n = 1 if kind < 0.2 else rng.randrange(2, 60) if kind < 0.35 else rng.randrange(65, 1400)
        segs.append((s, start, n))
    ctxs = [st + n for _, st, n in segs]
    # cache
    per = [-(-c // page) for c in ctxs]; n_pages = sum(per) + 3
    cache = torch.full((n_pages, 2, KV, page, hd), float("nan"), dtype=torch.bfloat16, device=dev)
    perm = torch.randperm(n_pages)[: sum(per)].tolist()
    table = torch.full((R, max(per)), -1, dtype=torch.int32)
    K, V = [], []
    it = iter(perm)
    for s, c in enumerate(ctxs):
        k = (0.7 * torch.randn(c, KV, hd, device=dev)).bfloat16(); v = torch.randn(c, KV, hd, device=dev).bfloat16()
        K.append(k); V.append(v)
        gone_before = max(0, segs[s][1] - window + 1) if window else 0
        for pi in range(per[s]):
            pg = next(it)
            if (pi + 1) * page <= gone_before: continue                 # the window has given this page back
            table[s, pi] = pg
            lo, hi = pi * page, min(c, (pi + 1) * page)
            blockk = torch.zeros(page, KV, hd, dtype=torch.bfloat16, device=dev); blockv = torch.zeros_like(blockk)
            blockk[: hi - lo] = k[lo:hi]; blockv[: hi - lo] = v[lo:hi]
            cache[pg, 0] = blockk.permute(1, 0, 2)
            cache[pg, 1].view(KV, hd, page).copy_(blockv.permute(1, 2, 0))
    table = table.to(dev)
    rows, seg_start, seg_len, seg_pos0, seg_slot = [], [], [], [], []
    for s, st, n in segs:
        seg_start.append(len(rows)); seg_len.append(n); seg_pos0.append(st); seg_slot.append(s)
        rows += [(s, st + i) for i in range(n)]
    T = len(rows)
    q = torch.randn(T, H * hd, device=dev).bfloat16()
    pos = torch.tensor([p for _, p in rows], dtype=torch.int32, device=dev); slots = torch.tensor([s for s, _ in rows], dtype=torch.int32, device=dev)
    ctx = StepContext(n_rows=T, dtype=torch.bfloat16, device=torch.device(dev), tokens=pos, row_pos=pos, row_slot=slots, seg_slot=seg_slot, seg_start=seg_start, seg_len=seg_len, seg_pos0=seg_pos0)
    out = torch.full((T, H * hd), float("nan"), dtype=torch.bfloat16, device=dev)
    ops.attention(q, cache, out, ctx, table, H, KV, hd, window)
    want = dense_ref(q, K, V, rows, H, KV, hd, window)
    err = float((out.double() - want).abs().max() / want.abs().max())
    assert bool(torch.isfinite(out.float()).all()) and err < 8e-3, f"case {case}: hd {hd} heads {H}:{KV} page {page} window {window} segments {segs}: {err}"
