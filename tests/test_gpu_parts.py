"""Each part of a layer alone against the plain functions, and a toy architecture defined in the
tests (windowed and full attention, a mixer with state of its own, a layer run twice, a layer that
reads another's cache) built and stepped through the framework as it is."""
import random

import pytest
import torch

import toy_architecture as toy
import traces
from model_folders import assert_within_bfloat16_noise, relative_error
from plain_llama import causal_attention, read_model_folder, rms_norm, rope_inverse_frequencies, rope_rotate, swiglu

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def step_context(segs, dtype):
    """segs: (slot, pos0, n) per request."""
    from geneinfer_amd.parts import StepContext
    pos, slots, seg_start = [], [], []
    for slot, pos0, n in segs:
        seg_start.append(len(pos))
        pos += list(range(pos0, pos0 + n))
        slots += [slot] * n
    t = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    return StepContext(n_rows=len(pos), dtype=dtype, device=torch.device(DEV), tokens=t(pos), row_pos=t(pos), row_slot=t(slots),
                       seg_slot=[s for s, _, _ in segs], seg_start=seg_start, seg_len=[n for _, _, n in segs], seg_pos0=[p for _, p, _ in segs])


def randn(*shape, seed=0, scale=1.0):
    return scale * torch.randn(*shape, generator=torch.Generator().manual_seed(seed))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_norm_part(dtype):
    from geneinfer_amd.config import RmsNormSpec
    from geneinfer_amd.parts import norm_class
    spec = RmsNormSpec(size=72, eps=0.02, weight="n.w")
    w = (1 + 0.1 * randn(72, seed=1)).to(dtype)
    part = norm_class(spec)(spec, {"n.w": w.to(DEV)}, dtype, DEV)
    assert [(n.name, n.shape, n.role) for n in part.tensor_needs(spec)] == [("n.w", (72,), "norm")]
    x = randn(9, 72, seed=2, scale=4.0)
    got = part(x.to(DEV), dtype)
    assert got.dtype == dtype and relative_error(got, rms_norm(x.double(), w.double(), 0.02)) < (2e-6 if dtype == torch.float32 else 5e-3)


def test_rotary_part_tables_are_shared_within_a_step():
    from geneinfer_amd.config import Llama3Scaling, RotarySpec
    from geneinfer_amd.config.llama import rotary_frequencies
    from geneinfer_amd.parts import position_class
    spec = RotarySpec(32, 500000.0, rotary_frequencies(32, 500000.0, Llama3Scaling(4.0, 1.0, 4.0, 32)))
    part = position_class(spec)(spec, {}, torch.float32, DEV)
    ctx = step_context([(0, 35, 4), (1, 0, 1)], torch.float32)
    cos, sin = part.half_split_tables(ctx)
    inv = rope_inverse_frequencies(32, 500000.0, dict(factor=4.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=32))
    ang = ctx.row_pos.cpu().double()[:, None] * inv[None, :]
    assert (cos.cpu().double() - ang.cos()).abs().max() < 1e-7 and (sin.cpu().double() - ang.sin()).abs().max() < 1e-7
    again = position_class(spec)(spec, {}, torch.float32, DEV).half_split_tables(ctx)
    assert again[0] is cos                                            # a second layer with the same spec reuses the step's tables


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [None, 5])
def test_attention_part_over_two_steps(dtype, window):
    """A portion, then its continuation beside another request's first rows: the part alone with a cache manager."""
    from geneinfer_amd.cache import CacheManager
    from geneinfer_amd.config import AttentionSpec, RotarySpec
    from geneinfer_amd.parts import LayerCache, mixer_class
    D, H, KV, hd = 40, 4, 2, 32
    spec = AttentionSpec(D, H, KV, hd, "q", "k", "v", "o", position=RotarySpec(hd, 10000.0), window=window)
    w = {"q": randn(H * hd, D, seed=1, scale=0.2), "k": randn(KV * hd, D, seed=2, scale=0.2), "v": randn(KV * hd, D, seed=3, scale=0.2),
         "o": randn(D, H * hd, seed=4, scale=0.2)}
    w = {k: v.to(dtype) for k, v in w.items()}
    cls = mixer_class(spec)
    part = cls(spec, {k: v.to(DEV) for k, v in w.items()}, dtype, DEV)
    assert {n.name: n.shape for n in cls.tensor_needs(spec)} == {"q": (128, 40), "k": (64, 40), "v": (64, 40), "o": (40, 128)}
    need = cls.cache_need(spec)
    assert (need.n_kv_heads, need.head_dim, need.window) == (KV, hd, window)
    cache = CacheManager([need], [None], page_size=16, n_pages=6, max_requests=2, max_positions=64, dtype=dtype, device=DEV)
    kv, table, _ = cache.kv(0)
    hs = {"a": randn(23, D, seed=5).to(dtype), "b": randn(7, D, seed=6).to(dtype)}
    got = {"a": [], "b": []}
    for step in ([("a", 0, 17)], [("a", 17, 6), ("b", 0, 7)]):
        for r, _, _ in step:
            if not cache.is_open(r):
                cache.open(r)
        cache.reserve([(r, n) for r, _, n in step]); cache.sync()
        ctx = step_context([(cache.slot(r), p0, n) for r, p0, n in step], dtype)
        h = torch.cat([hs[r][p0:p0 + n] for r, p0, n in step]).to(DEV)
        residual = torch.zeros(h.shape[0], D, device=DEV)
        part.forward(h, residual, ctx, LayerCache(kv=kv, table=table, writes=True))
        row = 0
        for r, _, n in step:
            got[r].append(residual[row:row + n].cpu()); row += n
            cache.advance(r, n)
    inv = rope_inverse_frequencies(hd, 10000.0)
    store = (lambda t: t.to(torch.bfloat16).double()) if dtype == torch.bfloat16 else (lambda t: t)
    for r, h in hs.items():
        T, hx = h.shape[0], h.double()
        wd = {k: v.double() for k, v in w.items()}
        q = store(rope_rotate((hx @ wd["q"].T).reshape(T, H, hd), torch.arange(T), inv))
        k = store(rope_rotate((hx @ wd["k"].T).reshape(T, KV, hd), torch.arange(T), inv))
        v = store((hx @ wd["v"].T).reshape(T, KV, hd))
        want = store(causal_attention(q, k, v, window)).reshape(T, H * hd) @ wd["o"].T
        assert relative_error(torch.cat(got[r]), want) < (3e-6 if dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_mixer_of_ones_own_uses_the_attention_front_half_with_a_hook(dtype):
    """An attention-like mixer defined here (it scales every query head and every key head by a number of its own before
    the rotation, as a per-head norm would) calls `qkv_rotate_store_attend` with that hook and gets the framework's kernels
    for product, rotation, page write and attention: a portion of 40 rows (tiles), then single rows (the kernel that
    rotates, stores and attends from the 32-bit products), against the plain functions."""
    from geneinfer_amd.cache import CacheManager, PagedKvNeed
    from geneinfer_amd.config import RotarySpec
    from geneinfer_amd.kernels import ops
    from geneinfer_amd.parts import LayerCache, position_class, qkv_rotate_store_attend
    D, H, KV, hd = 128, 4, 2, 64
    q_scale, k_scale = [0.5, 1.5, -1.0, 2.0], [1.25, 0.75]
    rot = RotarySpec(hd, 10000.0)
    position = position_class(rot)(rot, {}, dtype, DEV)
    w = {"q": randn(H * hd, D, seed=1, scale=0.2), "k": randn(KV * hd, D, seed=2, scale=0.2), "v": randn(KV * hd, D, seed=3, scale=0.2)}
    w = {k: v.to(dtype) for k, v in w.items()}
    w_qkv = torch.cat([w["q"], w["k"], w["v"]]).to(DEV).contiguous()
    calls = []

    def per_head(q, k):
        calls.append((tuple(q.shape), None if k is None else tuple(k.shape)))
        for h, c in enumerate(q_scale):
            ops.scale_rows(q[:, h * hd:(h + 1) * hd], c)
        for g, c in enumerate(k_scale):
            ops.scale_rows(k[:, g * hd:(g + 1) * hd], c)

    cache = CacheManager([PagedKvNeed(KV, hd, None)], [None], page_size=16, n_pages=4, max_requests=1, max_positions=64, dtype=dtype, device=DEV)
    kv, table, _ = cache.kv(0)
    T = 44
    hs = randn(T, D, seed=5).to(dtype)
    cache.open("a")
    got, fed = [], 0
    for n in (40, 1, 1, 2):
        cache.reserve([("a", n)]); cache.sync()
        ctx = step_context([(cache.slot("a"), fed, n)], dtype)
        att = qkv_rotate_store_attend(hs[fed:fed + n].to(DEV), w_qkv, ctx, LayerCache(kv=kv, table=table, writes=True), n_heads=H, n_kv_heads=KV,
                                      head_dim=hd, position=position, before_rotation=per_head)
        got.append(att.float().cpu())
        cache.advance("a", n)
        fed += n
    assert calls == [((n, H * hd), (n, KV * hd)) for n in (40, 1, 1, 2)]
    inv = rope_inverse_frequencies(hd, 10000.0)
    store = (lambda t: t.to(torch.bfloat16).double()) if dtype == torch.bfloat16 else (lambda t: t)
    hx, wd = hs.double(), {k: v.double() for k, v in w.items()}
    q = (hx @ wd["q"].T).reshape(T, H, hd) * torch.tensor(q_scale, dtype=torch.float64)[None, :, None]
    k = (hx @ wd["k"].T).reshape(T, KV, hd) * torch.tensor(k_scale, dtype=torch.float64)[None, :, None]
    q, k = store(rope_rotate(q, torch.arange(T), inv)), store(rope_rotate(k, torch.arange(T), inv))
    want = causal_attention(q, k, store((hx @ wd["v"].T).reshape(T, KV, hd))).reshape(T, H * hd)
    assert relative_error(torch.cat(got), want) < (3e-6 if dtype == torch.float32 else 1e-2)


def test_attention_refuses_a_head_size_its_kernels_do_not_take():
    from geneinfer_amd.config import AttentionSpec
    from geneinfer_amd.parts import mixer_class
    spec = AttentionSpec(64, 1, 1, 272, "q", "k", "v", "o")
    w = {"q": torch.zeros(272, 64, device=DEV), "k": torch.zeros(272, 64, device=DEV), "v": torch.zeros(272, 64, device=DEV), "o": torch.zeros(64, 272, device=DEV)}
    with pytest.raises(ValueError, match="head_dim = 272"):
        mixer_class(spec)(spec, w, torch.float32, DEV)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_feed_forward_part(dtype):
    from geneinfer_amd.config import SwiGluSpec
    from geneinfer_amd.parts import feed_forward_class
    D, I = 40, 112
    spec = SwiGluSpec(D, I, "g", "u", "d")
    w = {"g": randn(I, D, seed=1, scale=0.3).to(dtype), "u": randn(I, D, seed=2, scale=0.3).to(dtype), "d": randn(D, I, seed=3, scale=0.3).to(dtype)}
    part = feed_forward_class(spec)(spec, {k: v.to(DEV) for k, v in w.items()}, dtype, DEV)
    for rows in (1, 5, 70):                                           # decode-sized and prompt-sized batches take different kernels
        h = randn(rows, D, seed=rows).to(dtype)
        base = randn(rows, D, seed=rows + 1)
        residual = base.clone().to(DEV)
        part.forward(h.to(DEV), residual, step_context([(0, 0, rows)], dtype), )
        store = (lambda t: t.to(torch.bfloat16).double()) if dtype == torch.bfloat16 else (lambda t: t)
        want = base.double() + swiglu(h.double(), w["g"].double(), w["u"].double(), w["d"].double(), store)
        assert relative_error(residual, want) < (3e-6 if dtype == torch.float32 else 8e-3), rows


def test_registries_refuse_unknown_kinds_and_double_registration():
    from geneinfer_amd.parts import Mixer, mixer_class, register_mixer
    class Nothing:
        kind = "no_such_mixer"
    with pytest.raises(KeyError, match="no mixer of kind 'no_such_mixer' is registered; known: .*attention"):
        mixer_class(Nothing())
    with pytest.raises(ValueError, match="already registered"):
        register_mixer("attention", Mixer)


# ------------------------------------------------------------------------------------ toy model
# Two toy configurations that differ in every size and constant.  The second has heads of 32 channels, which the
# matrix-core attention kernels take in bfloat16 with pages of 16 positions: its windowed layer then feeds those
# kernels page tables with entries that the window has given back.
TOYS = {"small": (toy.ToyConfig(), [40, 9, 63, 21, 34], 5),
        "wide": (toy.ToyConfig(hidden_size=64, intermediate_size=96, num_attention_heads=4, num_key_value_heads=2, head_dim=32, vocab_size=173,
                               window=20, decay=0.6, angle_step=0.03, rotary_dim=20, embedding_scale=0.8, logit_cap=5.0, num_experts=2,
                               expert_intermediate_size=40, rms_norm_eps=3e-6, max_position_embeddings=320), [40, 9, 150, 21, 100], 6)}


@pytest.fixture(scope="module", params=list(TOYS))
def toy_model(request, tmp_path_factory):
    from geneinfer_amd.weights import write_random_model
    toy.register()
    toy.register()                                                    # registering the same classes again is harmless
    cfg, lengths, seed = TOYS[request.param]
    folder = tmp_path_factory.mktemp("toy")
    write_random_model(folder, cfg, seed=seed, dtype="bfloat16", std=0.2)
    _, weights = read_model_folder(folder)
    rng = random.Random(4)
    requests = {f"t{i}": [rng.randrange(cfg.vocab_size) for _ in range(n)] for i, n in enumerate(lengths)}
    # the routed feed-forward is exercised: every expert is some row's choice, and no choice hangs on the last digits
    top2 = torch.cat([torch.topk(toy.router_logits(cfg, weights, toks), 2, dim=-1).values for toks in requests.values()])
    chosen = torch.cat([toy.router_logits(cfg, weights, toks).argmax(-1) for toks in requests.values()])
    assert set(chosen.tolist()) == set(range(cfg.num_experts)) and float((top2[:, 0] - top2[:, 1]).min()) > 1e-4
    return cfg, folder, weights, requests


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", ["whole", "tail_singly", "portions", "long_portions", "mixed"])
def test_toy_architecture_under_every_cut(toy_model, dtype, mode):
    from geneinfer_amd.cache import PagedKvNeed, StateNeed
    from geneinfer_amd.engine import Runner, StepEntry, load_model
    from geneinfer_amd.parts import weight_bytes
    cfg, folder, weights, requests = toy_model
    model = load_model(folder, dtype, DEV)                            # config.json names the toy architecture; nothing else does
    assert type(model.config) is toy.ToyConfig
    # portions of 40, 110, ... rows: a portion long enough for the tiled prompt kernel begins behind pages the window gave back
    steps = {"whole": traces.whole, "tail_singly": lambda r: traces.tail_singly(r, 32), "portions": traces.portions,
             "long_portions": lambda r: traces.portions(r, sizes=(40, 110, 70)), "mixed": lambda r: traces.mixed(r, seed=8)}[mode](requests)
    runner = Runner(model, page_size=16 if dtype == "bfloat16" else 4, max_tokens=traces.peak_tokens(steps, 16), max_requests=4)
    groups = runner.cache.groups
    assert [(g.need.window, g.entries) for g in groups] == [(None, [1, 4]), (cfg.window, [2])]      # entry 5 reads entry 2's pages
    assert list(runner.cache.states) == [0, 3] and runner.cache.state(3).shape == (4 + 1, cfg.hidden_size)      # both decay mixers; four request slots and the spare one
    # what a step reads of the weights is asked of the parts, whatever a block calls them: every tensor of the file but the
    # token table, the two attention layers that run twice counted twice
    by_layer = lambda l: sum(4 * t.numel() for n, t in weights.items() if n.startswith(f"layers.{l}."))
    in_float32 = sum(by_layer(l) for l in (3, 0, 1, 2, 0, 1)) + 4 * weights["final_norm"].numel() + 4 * weights["head"].numel()
    read = model.weight_bytes_read_per_step()
    assert read == in_float32 if dtype == "float32" else in_float32 // 2 <= read < in_float32
    where, got = traces.wanted_positions(steps), {}
    gave_back = 0
    for s in steps:
        for e in s["entries"]:
            if not runner.is_open(e["id"]):
                runner.open(e["id"])
        logits = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
        for row, key in zip(logits.cpu(), where[s["step"]]):
            got[key] = row
        gave_back += sum(int(groups[1].first_live[runner.cache.slot(r)]) > 0 for r in runner.cache.open_requests())
        for rid in s["end"]:
            runner.close(rid)
        runner.cache.check_consistency()
        held = [sum(len(g.held_pages(runner.cache.slot(r))) for r in runner.cache.open_requests()) for g in groups]
        assert held[1] <= len(runner.cache.open_requests()) * (2 + (cfg.window + 8) // runner.page_size + 1)     # windowed pages are given back
    assert gave_back > 0, "no request ever ran with pages that its window had given back"
    assert runner.cache.free_pages() == [g.pool.n_pages for g in groups]
    exact = {rid: toy.plain_logits(cfg, weights, toks) for rid, toks in requests.items()}
    if dtype == "float32":
        worst = max(relative_error(row, exact[rid][p]) for (rid, p), row in got.items())
        assert worst < 2e-5, worst
    else:
        rounded = {rid: toy.plain_logits(cfg, weights, toks, store=lambda t: t.to(torch.bfloat16).double()) for rid, toks in requests.items()}
        assert_within_bfloat16_noise(got, lambda k: exact[k[0]][k[1]], lambda k: rounded[k[0]][k[1]], mode)
    # Every toy part reads what changes from step to step on the device (the decay mixer its state's slot, too), so the
    # steps of this model are captured like Llama's: the decode steps of a request's tail, and shapes that come again.
    assert runner.use_graphs is True
    if mode == "tail_singly":
        assert runner._graphs and all(g.graph is not None for g in runner._graphs.values()) and runner.steps_replayed >= 100


def test_a_part_whose_shapes_follow_the_data_switches_capturing_off(toy_model, monkeypatch):
    """The routed feed-forward that takes each expert's rows out (shapes that depend on the routing) says graph_safe = False:
    the runner then launches every step anew, and the logits are the same."""
    from geneinfer_amd.engine import Runner, StepEntry, load_model
    cfg, folder, weights, requests = toy_model
    monkeypatch.setattr(toy.RoutedFeedForward, "gathered", True)
    model = load_model(folder, "float32", DEV)
    assert model.graph_safe is False
    runner = Runner(model, page_size=4, max_tokens=256, max_requests=2)
    assert runner.use_graphs is False
    toks = requests["t3"]
    runner.open("a")
    runner.step([StepEntry("a", toks[:-4], ())])
    exact = toy.plain_logits(cfg, weights, toks)
    for i in range(len(toks) - 4, len(toks)):
        got = runner.step([StepEntry("a", [toks[i]], (0,))])[0].cpu()
        assert relative_error(got, exact[i]) < 2e-5
    assert not runner._graphs and runner.steps_replayed == 0
    runner.close("a")
    runner.cache.check_consistency()


def test_a_pass_that_raises_leaves_state_and_lengths_as_they_were(toy_model):
    """The second decay mixer of the run order fails once, after the first one has written its state: the step raises, the
    state slots and the request's length are what they were, and the same step then gives the logits of an undisturbed run."""
    from geneinfer_amd.engine import Runner, StepEntry, load_model
    cfg, folder, weights, requests = toy_model
    toks = requests["t0"]
    model = load_model(folder, "float32", DEV)
    runner = Runner(model, page_size=4, max_tokens=256, max_requests=2)
    runner.open("a")
    runner.step([StepEntry("a", toks[:7], ())])
    before = {e: s.clone() for e, s in runner.cache.states.items()}
    late = model.layers[2].mixer                                      # runs after layer 3's mixer (run-order entry 0)
    def failing(h, residual, ctx, cache):
        raise RuntimeError("no luck")
    late.forward = failing
    with pytest.raises(RuntimeError, match="no luck"):
        runner.step([StepEntry("a", toks[7:12], (4,))])
    del late.forward
    assert runner.length("a") == 7 and all(torch.equal(s, before[e]) for e, s in runner.cache.states.items())
    got = runner.step([StepEntry("a", toks[7:12], (4,))])[0].cpu()
    assert relative_error(got, toy.plain_logits(cfg, weights, toks[:12])[11]) < 2e-5
    runner.close("a")
    runner.cache.check_consistency()
