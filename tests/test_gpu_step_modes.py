"""The engine against the plain implementation, in 32-bit and in bfloat16, under every way of
cutting the work into steps.  In 32-bit the ways of cutting must also agree with each other bit
for bit: the 32-bit kernels sum in an order that does not depend on the batch."""
import random

import pytest
import torch

import traces
from model_folders import CONFIGS, PAGE_SIZE, assert_within_bfloat16_noise, relative_error, write_model
from plain_llama import PlainLlama

pytestmark = pytest.mark.gpu

# float32 is compared with the plain model in 64-bit.  bfloat16 is held against the rounding noise
# of a plain model that rounds to bfloat16 where the engine stores bfloat16 (see
# `assert_within_bfloat16_noise`).
TOLERANCE = {"float32": 2e-5}
LENGTHS = {"A": [5, 11, 17, 70, 45], "B": [1, 9, 33, 40, 75, 51], "C": [3, 66, 37, 50], "D": [150, 300, 37, 90, 700]}


def make_requests(name, seed=5):
    rng = random.Random(seed)
    vocab = CONFIGS[name]["vocab_size"]
    return {f"r{i}": [rng.randrange(vocab) for _ in range(n)] for i, n in enumerate(LENGTHS[name])}


@pytest.fixture(scope="module", params=["A", "B", "C", "D"])
def case(request, tmp_path_factory):
    name = request.param
    folder = tmp_path_factory.mktemp(f"tiny{name}")
    write_model(folder, CONFIGS[name], seed=11 + ord(name))
    requests = make_requests(name)
    plain, rounded = PlainLlama(folder), PlainLlama(folder, storage=torch.bfloat16)
    want = {"float32": {rid: plain.logits(toks) for rid, toks in requests.items()},
            "bfloat16": {rid: rounded.logits(toks) for rid, toks in requests.items()}}
    return name, folder, requests, want


def replay(folder, dtype, steps, page_size, max_tokens):
    from geneinfer_amd.engine import Runner, StepEntry, load_model
    model = load_model(folder, dtype, "cuda:0")
    runner = Runner(model, page_size=page_size, max_tokens=max_tokens, max_requests=4, max_rows=4096)
    got = {}
    where = traces.wanted_positions(steps)
    for s in steps:
        for e in s["entries"]:
            if not runner.is_open(e["id"]):
                runner.open(e["id"])
        logits = runner.step([StepEntry(e["id"], e["tokens"], e["want"]) for e in s["entries"]])
        if logits is not None:
            assert logits.shape[0] == len(where[s["step"]])
            for row, key in zip(logits.cpu(), where[s["step"]]):
                got[key] = row
        for rid in s["end"]:
            runner.close(rid)
    runner.cache.check_consistency()
    assert all(f == g.pool.n_pages for f, g in zip(runner.cache.free_pages(), runner.cache.groups)), "pages were not all given back"
    return got


def check(got, want, dtype):
    assert got, "the trace wanted no logits"
    worst = 0.0
    for (rid, pos), row in got.items():
        worst = max(worst, relative_error(row, want[rid][pos]))
    assert worst < TOLERANCE[dtype], f"worst relative error {worst:.3e}"
    return worst


_WHOLE = {}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", ["whole", "tail_singly", "portions", "mixed", "mixed_long"])
def test_step_modes(case, dtype, mode):
    name, folder, requests, want = case
    ps = PAGE_SIZE[name]
    if mode == "whole":
        steps = traces.whole(requests)
    elif mode == "tail_singly":
        steps = traces.tail_singly(requests, 32)
    elif mode == "portions":
        steps = traces.portions(requests)
    elif mode == "mixed":
        steps = traces.mixed(requests, seed=3)
        assert max(len(s["entries"]) for s in steps) >= 3, "the mixed trace never held three requests in a step"
    else:                                                        # portions of 70..200 rows: with tiny D, matrix-core tiles beside decoded rows
        steps = traces.mixed(requests, seed=5, portion=(70, 200), prompt_share=0.8)
        if name == "D":
            assert any(max(len(e["tokens"]) for e in s["entries"]) > 64 and min(len(e["tokens"]) for e in s["entries"]) == 1 for s in steps)
    max_tokens = traces.peak_tokens(steps, round_to=ps)          # so few pages that they are used again
    got = replay(folder, dtype, steps, ps, max_tokens)
    assert len(got) == sum(len(t) for t in requests.values())
    if dtype == "float32":
        worst = check(got, want[dtype], dtype)
        print(f"{name} {dtype} {mode}: worst relative error {worst:.2e}, {len(steps)} steps, pool of {max_tokens} positions")
    else:
        mean_e, mean_n = assert_within_bfloat16_noise(got, lambda k: want["float32"][k[0]][k[1]], lambda k: want["bfloat16"][k[0]][k[1]], f"{name} {mode}")
        print(f"{name} {dtype} {mode}: mean error {mean_e:.2e} (rounding noise {mean_n:.2e}), {len(steps)} steps, pool of {max_tokens} positions")
    if dtype == "float32":
        ref = _WHOLE.setdefault((name, "ref"), got if mode == "whole" else replay(folder, dtype, traces.whole(requests), ps, 4096))
        for key, row in got.items():
            assert torch.equal(row, ref[key]), f"{mode}: logits of {key} differ in bits from the whole-prompt run"


def test_changing_first_token_changes_logits(case):
    """The comparison is not vacuous: another first token gives other logits at the last position."""
    name, folder, requests, want = case
    rid = "r2"
    toks = list(requests[rid])
    toks[0] = (toks[0] + 1) % CONFIGS[name]["vocab_size"]
    got = replay(folder, "float32", traces.whole({rid: toks}), PAGE_SIZE[name], 4096)
    assert relative_error(got[(rid, len(toks) - 1)], want["float32"][rid][len(toks) - 1]) > 1e-3


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_rewind_and_go_another_way(case, dtype):
    """A request is cut back (inside a page, at a page's edge, to nothing) and fed other tokens: the logits are
    those of the sequence as it now stands.  One rewind falls into a page that a second request shares; that
    request's later logits do not change."""
    from geneinfer_amd.engine import Runner, StepEntry, load_model
    name, folder, requests, _ = case
    ps, vocab = PAGE_SIZE[name], CONFIGS[name]["vocab_size"]
    rng = random.Random(77)
    base = [rng.randrange(vocab) for _ in range(3 * ps + 3)]
    plain, rounded = PlainLlama(folder), PlainLlama(folder, storage=torch.bfloat16)
    model = load_model(folder, dtype, "cuda:0")
    runner = Runner(model, page_size=ps, max_tokens=16 * ps, max_requests=2, max_rows=4096)
    assert runner.cache.enable_prefix_sharing()
    runner.open("a")
    runner.step([StepEntry("a", base, ())])
    runner.cache.prefix.insert(base, len(base), runner.cache.pages_of("a"))
    runner.open("b", runner.cache.prefix.match(base, len(base) - 1))          # b shares a's three full pages
    assert runner.length("b") == 3 * ps
    got, exact, near = {}, {}, {}
    def feed(rid, history, tokens):
        rows = runner.step([StepEntry(rid, tokens, tuple(range(len(tokens))))]).cpu()
        now = history + tokens
        e, r = plain.logits(now), rounded.logits(now)
        for i, row in enumerate(rows):
            key = (rid, len(got))
            got[key], exact[key], near[key] = row, e[len(history) + i], r[len(history) + i]
        return now
    seq_b = feed("b", base[:3 * ps], base[3 * ps:3 * ps + 2])
    seq_a = list(base)
    for cut in (2 * ps + 3, 2 * ps, ps - 1, 0):                                 # the first falls into a page that b shares
        runner.truncate("a", cut)
        assert runner.length("a") == cut
        other = [rng.randrange(vocab) for _ in range(ps + 2)]
        seq_a = feed("a", seq_a[:cut], other[:1])                               # one token through the decode path
        seq_a = feed("a", seq_a, other[1:])                                     # then a portion
        runner.cache.check_consistency()
    assert set(runner.cache.pages_of("a")).isdisjoint(runner.cache.pages_of("b")[:3])
    feed("b", seq_b, base[3 * ps + 2:])                                         # b still reads the pages as a first wrote them
    if dtype == "float32":
        worst = max(relative_error(row, exact[key]) for key, row in got.items())
        assert worst < TOLERANCE["float32"], f"worst relative error {worst:.3e}"
    else:
        assert_within_bfloat16_noise(got, exact.__getitem__, near.__getitem__, f"tiny {name}, rewind")
    runner.close("a"); runner.close("b")
    runner.cache.prefix.clear()
    runner.cache.check_consistency()
    assert runner.cache.free_pages() == [g.pool.n_pages for g in runner.cache.groups]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_steps_whose_shape_comes_again_are_replayed_from_a_captured_pass(tmp_path, dtype):
    """Tiny D: three requests decode while a fourth's prompt goes in as portions of 96 rows, the same shape step after step
    (captured at its second coming, replayed from then on), then alone in portions of 130 rows; every decoded row's logits and
    each portion's last are the plain model's, and in 32-bit equal in bits to those of a runner that captures no such step."""
    from geneinfer_amd.engine import Runner, StepEntry, load_model
    write_model(tmp_path, CONFIGS["D"], seed=3)
    rng = random.Random(8)
    vocab = CONFIGS["D"]["vocab_size"]
    short = {f"s{i}": [rng.randrange(vocab) for _ in range(30 + 7 * i + 8)] for i in range(3)}      # prompts of 30, 37, 44, then 8 single tokens
    long = {"p": [rng.randrange(vocab) for _ in range(8 * 96)], "q": [rng.randrange(vocab) for _ in range(5 * 130)]}
    plain = PlainLlama(tmp_path)
    exact = {r: plain.logits(t) for r, t in {**short, **long}.items()}
    near = {r: plain.with_storage(torch.bfloat16).logits(t) for r, t in {**short, **long}.items()}
    model = load_model(tmp_path, dtype, "cuda:0")

    def run(graph_rows):
        runner = Runner(model, page_size=16, max_tokens=2048, max_requests=4, max_rows=1024, graph_rows=graph_rows)
        got, fed = {}, {}
        for r, toks in short.items():
            runner.open(r)
            runner.step([StepEntry(r, toks[:len(toks) - 8], ())])
            fed[r] = len(toks) - 8
        runner.open("p")
        for k in range(8):                                            # (1, 1, 1, 96) eight times
            entries = [StepEntry(r, [short[r][fed[r]]], (0,)) for r in short] + [StepEntry("p", long["p"][96 * k:96 * k + 96], (95,))]
            rows = runner.step(entries).cpu()
            for i, r in enumerate(short):
                got[(r, fed[r])] = rows[i]
                fed[r] += 1
            got[("p", 96 * k + 95)] = rows[3]
        for r in list(short) + ["p"]:
            runner.close(r)
        runner.open("q")
        for k in range(5):                                            # (130,) five times: tiles of 64 rows, in pairs
            got[("q", 130 * k + 129)] = runner.step([StepEntry("q", long["q"][130 * k:130 * k + 130], (129,))])[0].cpu()
        runner.close("q")
        runner.cache.check_consistency()
        return got, runner

    got, runner = run(1024)
    shapes = {key[0]: g for key, g in runner._step_graphs.items()}
    assert shapes[(1, 1, 1, 96)].graph is not None and shapes[(1, 1, 1, 96)].calls == 8, "the mixed step's shape was not captured and replayed"
    assert shapes[(130,)].graph is not None and shapes[(130,)].calls == 5
    if dtype == "float32":
        worst = max(relative_error(row, exact[r][p]) for (r, p), row in got.items())
        assert worst < TOLERANCE["float32"], f"worst relative error {worst:.3e}"
        plainly, other = run(0)
        assert not other._step_graphs
        for key, row in got.items():
            assert torch.equal(row, plainly[key]), f"logits of {key} differ in bits between the captured step and the step run as it is"
    else:
        assert_within_bfloat16_noise(got, lambda k: exact[k[0]][k[1]], lambda k: near[k[0]][k[1]], "tiny D, captured steps")


def test_a_runner_with_captured_steps_is_freed_without_the_cycle_collector(case):
    """A runner and its captured graphs form no reference cycle: dropping the runner frees them at once, not at a
    moment of the cycle collector's choosing (which may fall inside another capture, where freeing aborts)."""
    import gc
    import weakref
    from geneinfer_amd.engine import Runner, StepEntry, load_model
    name, folder, requests, _ = case
    model = load_model(folder, "bfloat16", "cuda:0")
    gc.collect()
    gc.disable()
    try:
        runner = Runner(model, page_size=PAGE_SIZE[name], max_tokens=256, max_requests=2, max_rows=64)
        runner.open("a")
        runner.step([StepEntry("a", [1, 2, 3], (2,))])
        for t in (4, 5, 6):                                   # the second one-token step of a batch size is captured
            runner.step([StepEntry("a", [t], (0,))])
        (graph,) = runner._graphs.values()
        assert runner.use_graphs and graph.graph is not None
        graph_ref, runner_ref = weakref.ref(graph), weakref.ref(runner)
        del graph
        torch.cuda.synchronize()
        del runner
        assert runner_ref() is None and graph_ref() is None
    finally:
        gc.enable()
