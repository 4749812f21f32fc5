"""The engine against the plain implementation at the layer shape of Llama 3.2 1B (hidden 2048, 32 query heads over 8
key/value heads of 64 channels, feed-forward 8192, vocabulary 128256, llama3 scaling with factor 32, tied table, pages of
16), with 2 of the 16 layers: the kernel instances that the benchmark runs (the products' large tiles, the gated
feed-forward product over 2048 of k, the head over 128256 rows, prompt attention over many paired tiles, decode attention
with split contexts) meet the plain model under every way of cutting the work, in 32-bit and in bfloat16.  Logits are
compared at every 16th position and at the last of each request.  What tests/verify_forward.py:72-117 does for the
reference at its sizes.  The layer shape of Llama 3.2 3B (hidden 3072, 24 query heads over 8 key/value heads of 128
channels, one layer, a cut vocabulary) follows in bfloat16 under the cuts that differ most: whole prompts, and long
portions beside single tokens with pages used again."""
import random

import pytest
import torch

import traces
from model_folders import LLAMA_1B_SHAPE, LLAMA_3B_SHAPE, assert_within_bfloat16_noise, relative_error, write_model
from plain_llama import PlainLlama

pytestmark = pytest.mark.gpu
LENGTHS = [640, 40, 75, 130]
EVERY = 16
PAGE = 16


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
