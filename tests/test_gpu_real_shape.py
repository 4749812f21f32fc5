"""The engine against the plain implementation at the layer shape of Llama 3.2 1B (hidden 2048, 32 query heads over 8
key/value heads of 64 channels, feed-forward 8192, vocabulary 128256, llama3 scaling with factor 32, tied table, pages of
16), with 2 of the 16 layers: the kernel instances that the benchmark runs (the products' large tiles, the gated
feed-forward product over 2048 of k, the head over 128256 rows, prompt attention over many paired tiles, decode attention
with split contexts) meet the plain model under every way of cutting the work, in 32-bit and in bfloat16.  Logits are
compared at every 16th position and at the last of each request.  What tests/verify_forward.py:72-117 does for the
reference at its sizes.  The layer shape of Llama 3.2 3B (hidden 3072, 24 query heads over 8 key/value heads of 128
channels, one layer, a cut vocabulary) follows in bfloat16 under the cuts that differ most: whole prompts, and long
portions beside single tokens with pages used again.

Then the steps that serve many requests at once: 72 requests decode together, one token each, and close in groups, so that
steps of 72, 65, 64, 40, 24 and 17 rows run, each size three times (as it comes, captured, replayed), through the runner's
captured graphs with their fill rows, against the plain model row by row; and the same prompts through the scheduler with 64
running requests and steps queued ahead, against the single-request loop.  What tools/engine_check_main.cpp:179-211 does
for the reference: every request through the engine gets what it gets alone."""
import random

import pytest
import torch

import traces
from model_folders import (LLAMA_1B_SHAPE, LLAMA_3B_SHAPE, assert_within_bfloat16_noise, formula_weights, full_config, relative_error,
                           write_model)
from plain_llama import PlainLlama

pytestmark = pytest.mark.gpu
LENGTHS = [640, 40, 75, 130]
EVERY = 16
PAGE = 16


_PLAIN = {}                       # folder -> its plain model, kept for the tests that ask it about other requests


def make_case(folder, sizes, seed):
    write_model(folder, sizes, seed=seed, dtype=torch.bfloat16, std=0.02)
    rng = random.Random(9)
    requests = {f"r{i}": [rng.randrange(sizes["vocab_size"]) for _ in range(n)] for i, n in enumerate(LENGTHS)}
    plain = PlainLlama(folder)
    rounded = plain.with_storage(torch.bfloat16)
    want = {"float32": {}, "bfloat16": {}}
    for rid, toks in requests.items():
        places = [p for p in range(len(toks)) if p % EVERY == 0 or p == len(toks) - 1]
        for dtype, model in (("float32", plain), ("bfloat16", rounded)):
            for p, row in zip(places, model.logits_at(toks, places)):
                want[dtype][(rid, p)] = row
    _PLAIN[str(folder)] = plain
    return folder, requests, want, {}


@pytest.fixture(scope="module")
def case(tmp_path_factory):
    return make_case(tmp_path_factory.mktemp("llama1b_shape"), LLAMA_1B_SHAPE, 31)


@pytest.fixture(scope="module")
def case_3b(tmp_path_factory):
    return make_case(tmp_path_factory.mktemp("llama3b_shape"), LLAMA_3B_SHAPE, 32)


def model_of(case, dtype):
    from geneinfer_amd.engine import load_model
    folder, _, _, models = case
    if dtype not in models:
        models.clear()                                   # one model of this size at a time
        models[dtype] = load_model(folder, dtype, "cuda:0")
    return models[dtype]


def replay(model, steps, max_tokens):
    from geneinfer_amd.engine import Runner, StepEntry
    runner = Runner(model, page_size=PAGE, max_tokens=max_tokens, max_requests=4, max_rows=4096)
    got, where = {}, traces.wanted_positions(steps)
    for s in steps:
        for e in s["entries"]:
            if not runner.is_open(e["id"]):
                runner.open(e["id"])
        logits = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
        if logits is not None:
            for row, key in zip(logits.cpu(), where[s["step"]]):
                got[key] = row
        for rid in s["end"]:
            runner.close(rid)
    runner.cache.check_consistency()
    assert runner.cache.free_pages() == [g.pool.n_pages for g in runner.cache.groups], "pages were not all given back"
    return got


MODES = {"whole": lambda r: traces.whole(r, EVERY), "tail_singly": lambda r: traces.tail_singly(r, 32, EVERY),
         "portions": lambda r: traces.portions(r, want_every=EVERY),
         "long_portions": lambda r: traces.portions(r, sizes=(130, 2, 257, 70, 3), want_every=EVERY),
         "mixed": lambda r: traces.mixed(r, seed=4, want_every=EVERY),
         "mixed_long": lambda r: traces.mixed(r, seed=6, portion=(70, 200), prompt_share=0.8, want_every=EVERY)}
_WHOLE = {}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", list(MODES))
def test_llama_1b_layer_shape_under_every_cut(case, dtype, mode):
    folder, requests, want, _ = case
    steps = MODES[mode](requests)
    if mode.startswith("mixed"):
        assert max(len(s["entries"]) for s in steps) >= 2
    if mode == "mixed_long":                              # a prompt portion long enough for matrix-core tiles beside single decoded tokens
        assert any(max(len(e["tokens"]) for e in s["entries"]) > 64 and min(len(e["tokens"]) for e in s["entries"]) == 1 for s in steps)
    model = model_of(case, dtype)
    got = replay(model, steps, traces.peak_tokens(steps, round_to=PAGE))
    assert set(got) == set(want[dtype]), "the trace did not ask for the compared positions"
    if dtype == "float32":
        worst = max(relative_error(row, want["float32"][key]) for key, row in got.items())
        assert worst < 2e-5, f"worst relative error {worst:.3e}"
        ref = _WHOLE.setdefault("whole", got if mode == "whole" else replay(model, MODES["whole"](requests), 4096))
        for key, row in got.items():
            assert torch.equal(row, ref[key]), f"{mode}: logits of {key} differ in bits from the whole-prompt run"
        print(f"1B shape float32 {mode}: worst relative error {worst:.2e}, {len(steps)} steps")
    else:
        mean_e, mean_n = assert_within_bfloat16_noise(got, want["float32"].__getitem__, want["bfloat16"].__getitem__, f"1B shape, {mode}")
        print(f"1B shape bfloat16 {mode}: mean error {mean_e:.2e} (rounding noise {mean_n:.2e}), {len(steps)} steps")


@pytest.mark.parametrize("mode", ["whole", "tail_singly", "mixed_long"])
def test_llama_3b_layer_shape_in_bfloat16(case_3b, mode):
    folder, requests, want, _ = case_3b
    steps = MODES[mode](requests)
    model = model_of(case_3b, "bfloat16")
    got = replay(model, steps, traces.peak_tokens(steps, round_to=PAGE))
    assert set(got) == set(want["bfloat16"])
    mean_e, mean_n = assert_within_bfloat16_noise(got, want["float32"].__getitem__, want["bfloat16"].__getitem__, f"3B shape, {mode}")
    print(f"3B shape bfloat16 {mode}: mean error {mean_e:.2e} (rounding noise {mean_n:.2e}), {len(steps)} steps")


# ------------------------------------------------------------------------------------------------ many requests decoding at once
@pytest.mark.parametrize("length", [1600, 700])
def test_llama_1b_layer_shape_long_prompt_with_the_norms_inside_the_products(case, length):
    """A prompt of 1,600 tokens (and of 700, where the gated product's tiles of 256 x 256 reach three quarters of the compute
    units only) in one step, in bfloat16: at this many rows the products have the tiles whose last steps do the
    two norms of a layer between them (the output and down projections write g * x and the pieces of the rows' sums of squares,
    the q/k/v product and the gated product multiply by the rows' factors); every 64th position and the last against the
    plain model, and the norm's own kernel is called for the first layer's first norm and the final norm only."""
    from geneinfer_amd.engine import Runner, StepEntry
    from geneinfer_amd.kernels import ops
    folder, _, _, _ = case
    plain = _PLAIN[str(folder)]
    rng = random.Random(21)
    toks = [rng.randrange(LLAMA_1B_SHAPE["vocab_size"]) for _ in range(length)]
    places = [p for p in range(len(toks)) if p % 64 == 0] + [len(toks) - 1]
    model = model_of(case, "bfloat16")
    d, inter = LLAMA_1B_SHAPE["hidden_size"], LLAMA_1B_SHAPE["intermediate_size"]
    pieces = (d // 128,) if length == 1600 else (d // 128, d // 1024)      # (from the tiles' epilogues; with few tiles, from the kernel that adds the shares of k)
    assert ops.gemm_bf16_norm_parts(length, d, inter) in pieces and ops.gemm_bf16_norm_parts(length, d, d) in pieces
    assert ops.gemm_bf16_takes_norm(length, 2 * inter, d, True)
    runner = Runner(model, page_size=PAGE, max_tokens=1664, max_requests=1, max_rows=2048)
    runner.open("long")
    profile = ops.set_profiling(True)
    try:
        logits = runner.step([StepEntry("long", toks, places)]).cpu()
    finally:
        ops.set_profiling(False)
    runner.close("long")
    norms = sum(calls for label, calls in profile.calls.items() if label.startswith("rmsnorm"))
    exact = plain.logits_at(toks, places)
    rounded = plain.with_storage(torch.bfloat16).logits_at(toks, places)
    got = {("long", p): row for p, row in zip(places, logits)}
    want_exact = {("long", p): row for p, row in zip(places, exact)}
    want_rounded = {("long", p): row for p, row in zip(places, rounded)}
    mean_e, mean_n = assert_within_bfloat16_noise(got, want_exact.__getitem__, want_rounded.__getitem__, f"1B shape, {length}-token prompt")
    print(f"1B shape bfloat16 long prompt: mean error {mean_e:.2e} (rounding noise {mean_n:.2e}); norm kernels {norms}")
    assert norms == 2, profile.calls


WIDE_SIZES = [72, 65, 64, 40, 24, 17]          # rows of the all-decode steps, in this order
WIDE_STEPS_EACH = 3                            # a size runs as it comes, is captured at its second step, and replayed at its third


def wide_requests(vocab, seed=12):
    """72 requests: request i has a prompt of 20 to 60 tokens and then one given token for every step it lives through
    (it closes when the step size falls to i or below)."""
    rng = random.Random(seed)
    requests, alive = {}, {}
    for i in range(max(WIDE_SIZES)):
        alive[f"w{i}"] = WIDE_STEPS_EACH * sum(1 for n in WIDE_SIZES if n > i)
        requests[f"w{i}"] = [rng.randrange(vocab) for _ in range(rng.randint(20, 60) + alive[f"w{i}"])]
    return requests, alive


def wide_decode(model, requests, alive, use_graphs):
    """Prompts in steps of eight requests (nothing wanted), then the all-decode steps.  Returns {(request, position): logits row},
    and the runner."""
    from geneinfer_amd.engine import Runner, StepEntry
    ids = list(requests)
    pool = sum(-(-len(requests[r]) // PAGE) * PAGE for r in ids)                      # every request's final length, in whole pages: nothing to spare
    runner = Runner(model, page_size=PAGE, max_tokens=pool, max_requests=len(ids), max_rows=1024, use_graphs=use_graphs)
    fed = {}
    for first in range(0, len(ids), 8):
        group = ids[first:first + 8]
        for r in group:
            runner.open(r)
            fed[r] = len(requests[r]) - alive[r]
        runner.step([StepEntry(r, requests[r][:fed[r]], ()) for r in group])
    got = {}
    for size in WIDE_SIZES:
        for r in ids[size:]:
            if runner.is_open(r):
                assert fed[r] == len(requests[r])
                runner.close(r)
        live = ids[:size]
        for _ in range(WIDE_STEPS_EACH):
            logits = runner.step([StepEntry(r, [requests[r][fed[r]]], (0,)) for r in live]).cpu()
            for r, row in zip(live, logits):
                got[(r, fed[r])] = row
                fed[r] += 1
    for r in ids[:WIDE_SIZES[-1]]:
        runner.close(r)
    runner.cache.check_consistency()
    assert runner.cache.free_pages() == [g.pool.n_pages for g in runner.cache.groups], "pages were not all given back"
    return got, runner


_WIDE_WANT = {}


def wide_want(plain, requests, alive, storage=None):
    key = (id(plain), storage)
    if key not in _WIDE_WANT:
        _WIDE_WANT[key] = _wide_want(plain, requests, alive, storage)
    return _WIDE_WANT[key]


def _wide_want(plain, requests, alive, storage):
    model = plain if storage is None else plain.with_storage(storage)
    want = {}
    for r, toks in requests.items():
        places = list(range(len(toks) - alive[r], len(toks)))
        for p, row in zip(places, model.logits_at(toks, places)):
            want[(r, p)] = row.float()
    return want


def assert_wide_graphs(runner):
    """Which captured steps served the run: 72 rows (also for 65 requests, filled up), 64, 40, 24 and 20 (for 17)."""
    sizes = sorted(batch for batch, _ in runner._graphs)
    assert sizes == [20, 24, 40, 64, 72], f"captured batch sizes {sizes}"
    for (batch, bracket), g in runner._graphs.items():
        assert g.graph is not None and g.calls == WIDE_STEPS_EACH * (2 if batch == 72 else 1), f"the graph of {batch} rows was not captured and replayed"
    return sizes


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_llama_1b_layer_shape_many_requests_decode_at_once(case, dtype):
    folder, _, _, _ = case
    requests, alive = wide_requests(LLAMA_1B_SHAPE["vocab_size"])
    model = model_of(case, dtype)
    got, runner = wide_decode(model, requests, alive, use_graphs=True)
    sizes = assert_wide_graphs(runner)
    exact = wide_want(_PLAIN[str(folder)], requests, alive)
    assert set(got) == set(exact) and len(got) == WIDE_STEPS_EACH * sum(WIDE_SIZES)
    if dtype == "float32":
        worst = max(relative_error(row, exact[key]) for key, row in got.items())
        assert worst < 2e-5, f"worst relative error {worst:.3e}"
        plain_steps, other = wide_decode(model, requests, alive, use_graphs=False)
        assert not other._graphs
        for key, row in got.items():
            assert torch.equal(row, plain_steps[key]), f"logits of {key} differ in bits between the captured steps and steps run as they are"
        print(f"1B shape float32, steps of {WIDE_SIZES} rows through graphs of {sizes}: worst relative error {worst:.2e}")
    else:
        rounded = wide_want(_PLAIN[str(folder)], requests, alive, torch.bfloat16)
        mean_e, mean_n = assert_within_bfloat16_noise(got, exact.__getitem__, rounded.__getitem__, "1B shape, many requests decoding")
        print(f"1B shape bfloat16, steps of {WIDE_SIZES} rows through graphs of {sizes}: mean error {mean_e:.2e} (rounding noise {mean_n:.2e})")


def test_llama_3b_layer_shape_many_requests_decode_at_once(case_3b):
    folder, _, _, _ = case_3b
    requests, alive = wide_requests(LLAMA_3B_SHAPE["vocab_size"])
    got, runner = wide_decode(model_of(case_3b, "bfloat16"), requests, alive, use_graphs=True)
    sizes = assert_wide_graphs(runner)
    exact = wide_want(_PLAIN[str(folder)], requests, alive)
    rounded = wide_want(_PLAIN[str(folder)], requests, alive, torch.bfloat16)
    assert set(got) == set(exact)
    mean_e, mean_n = assert_within_bfloat16_noise(got, exact.__getitem__, rounded.__getitem__, "3B shape, many requests decoding")
    print(f"3B shape bfloat16, steps of {WIDE_SIZES} rows through graphs of {sizes}: mean error {mean_e:.2e} (rounding noise {mean_n:.2e})")


def test_llama_1b_layer_shape_scheduler_with_64_running_requests(case):
    """The 72 prompts through the scheduler, 64 running at a time, decode steps queued ahead of the host, graphs on: every
    request ends with the tokens the single-request loop gives it, bit for bit in 32-bit.  Requests generate 6 to 24 tokens,
    so the batch drains and the last eight are admitted as others finish."""
    import geneinfer_amd as gi
    from geneinfer_amd.engine import EngineConfig, EngineRequest
    from geneinfer_amd.sampling import SamplerConfig
    requests, alive = wide_requests(LLAMA_1B_SHAPE["vocab_size"])
    rng = random.Random(3)
    prompts = [toks[:len(toks) - alive[r]] for r, toks in requests.items()]
    new = [rng.randint(6, 24) for _ in prompts]
    llm = gi.LLM(model_of(case, "float32"), page_size=PAGE, max_tokens=64 * 96, max_running=64, max_rows=1024)
    alone = [llm.generate(p, steps=len(p) + n - 1, temperature=0.0).generated_tokens for p, n in zip(prompts, new)]
    assert [len(a) for a in alone] == new
    eng = llm.engine(EngineConfig(max_running=64, step_rows=512))
    ids = [eng.submit(EngineRequest(p, len(p) + n - 1, SamplerConfig(0.0))) for p, n in zip(prompts, new)]
    flights = 0
    while eng.step():
        flights += eng._flight is not None
    out = [eng.result(j) for j in ids]
    assert all(r.finished and r.error == "" for r in out)
    assert eng.stats.max_running_seen == 64 and flights > 10, "the scheduler did not run 64 requests with steps queued ahead"
    assert any(batch >= 40 for batch, _ in llm.runner._graphs), f"captured batch sizes {sorted(llm.runner._graphs)}"
    assert [r.generated_tokens for r in out] == alone
    llm.runner.cache.check_consistency()


def test_the_weights_the_benchmark_draws_can_be_remade_and_give_the_plain_logits(tmp_path):
    """`random_model(..., draw_on_device=True)`, what bench.py runs, at the 1B layer shape: the tensors on the device are, bit for
    bit, the ones this suite re-makes from the stated formula, and the model's bfloat16 logits for a prompt and decoded tokens
    are the plain model's on the re-made weights."""
    from geneinfer_amd.config import LlamaConfig
    from geneinfer_amd.engine import Runner, StepEntry, random_model
    sizes = dict(LLAMA_1B_SHAPE, num_hidden_layers=1)
    model = random_model(LlamaConfig.from_dict(sizes), seed=5, dtype="bfloat16", device="cuda:0", draw_on_device=True)
    remade = formula_weights(full_config(sizes), seed=5, std=0.02)
    assert torch.equal(model.embedding.cpu(), remade["model.embed_tokens.weight"].to(torch.bfloat16))
    layer = model.layers[0]
    assert torch.equal(layer.mixer.w_o.cpu(), remade["model.layers.0.self_attn.o_proj.weight"].to(torch.bfloat16))
    assert torch.equal(layer.mixer_norm.weight.cpu(), remade["model.layers.0.input_layernorm.weight"].to(torch.bfloat16))
    assert torch.equal(layer.feed_forward.w_down.cpu(), remade["model.layers.0.mlp.down_proj.weight"].to(torch.bfloat16))
    write_model(tmp_path, sizes, dtype=torch.bfloat16, weights=remade)
    plain = PlainLlama(tmp_path)
    rng = random.Random(2)
    toks = [rng.randrange(sizes["vocab_size"]) for _ in range(150)]
    places = list(range(0, 140, 20)) + list(range(140, 150))
    exact, rounded = plain.logits_at(toks, places), plain.with_storage(torch.bfloat16).logits_at(toks, places)
    runner = Runner(model, page_size=PAGE, max_tokens=160, max_requests=1, max_rows=256)
    runner.open("r")
    got = dict(zip(range(0, 140, 20), runner.step([StepEntry("r", toks[:140], tuple(range(0, 140, 20)))]).cpu()))
    for p in range(140, 150):
        got[p] = runner.step([StepEntry("r", [toks[p]], (0,))])[0].cpu()
    runner.close("r")
    at = {p: i for i, p in enumerate(places)}
    assert_within_bfloat16_noise(got, lambda p: exact[at[p]], lambda p: rounded[at[p]], "the benchmark's random model")
