"""Generation on the GPU: the single-request loop and the scheduler against each other and against
the plain implementation, sampling on the device, long decoding and the first tokens of a sequence."""
import random

import pytest
import torch

from model_folders import CONFIGS, PAGE_SIZE, assert_within_bfloat16_noise, relative_error, write_model
from plain_llama import PlainLlama
import plain_sampler

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    out = {}
    for name in ("A", "B", "D"):
        out[name] = tmp_path_factory.mktemp(f"gen{name}")
        write_model(out[name], CONFIGS[name], seed=40 + ord(name))
    return out


def prompts_for(name, lengths, seed=9):
    rng = random.Random(seed)
    return [[rng.randrange(CONFIGS[name]["vocab_size"]) for _ in range(n)] for n in lengths]


def test_greedy_generation_through_the_entry_point(folders):
    """Tiny A: prompts of 5, 11 and 17 tokens, 8 greedy tokens each, pages of 4 positions."""
    import geneinfer_amd as gi
    plain = PlainLlama(folders["A"])
    llm = gi.LLM(folders["A"], dtype="float32", page_size=PAGE_SIZE["A"], max_tokens=64, max_running=2)
    for prompt in prompts_for("A", [5, 11, 17]):
        got = llm.generate(prompt, steps=len(prompt) + 7, temperature=0.0)
        assert got.generated_tokens == plain.greedy(prompt, 8) and not got.stopped_by_end_token
        assert got.decode_steps == 7 and got.prefill_ms > 0
    assert llm.runner.cache.free_pages() == [16]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_profiling_times_every_kernel_and_changes_no_token(folders, dtype):
    """With the per-kernel timing on, no step is replayed from a graph and every kernel is waited for; the tokens are
    those of the unobserved run, the report names the kernels with their counts, and the products say whose weights
    they read.  Switched off, decoding is replayed from graphs again."""
    import geneinfer_amd as gi
    from geneinfer_amd.kernels import ops
    cfg = CONFIGS["B"]
    llm = gi.LLM(folders["B"], dtype=dtype, page_size=PAGE_SIZE["B"], max_tokens=128, max_running=2)
    prompt = prompts_for("B", [9])[0]
    assert llm.profile_report() == ""
    plain_run = llm.generate(prompt, steps=len(prompt) + 5, temperature=0.0).generated_tokens
    graphs = len(llm.runner._graphs)
    assert graphs >= 1 and llm.runner.can_step_from_device
    try:
        llm.set_profiling(True)
        assert not llm.runner.can_step_from_device
        steps_before = llm.runner.steps_run
        assert llm.generate(prompt, steps=len(prompt) + 5, temperature=0.0).generated_tokens == plain_run
        report = llm.profile_report()
    finally:
        llm.set_profiling(False)
    steps = llm.runner.steps_run - steps_before
    assert steps == 7 and f"device profile: {len(prompt) + 5} positions in 7 steps" in report      # the prompt but its last token, then one by one
    rows = {line[2:36].strip(): line[36:].split() for line in report.splitlines()[2:]}
    layers, hidden, inter = cfg["num_hidden_layers"], cfg["hidden_size"], cfg["intermediate_size"]
    product = "gemm_exact" if dtype == "float32" else "gemm_bf16"
    down = f"{product} {hidden}x{inter}"
    assert down in rows and int(rows[down][0]) == layers * steps and float(rows[down][-1]) > 0        # calls; weights GB/s
    assert f"{product} {cfg['vocab_size']}x{hidden}" in rows
    assert int(rows[f"{product} {cfg['vocab_size']}x{hidden}"][0]) == steps - 1                          # the head: not for the prompt, whose logits nobody wants
    assert any(k.startswith("attention") for k in rows) and ("embed" in rows or "embed_handing" in rows)
    # norm kernels: in 32-bit two a layer and the final one where logits are wanted; in bfloat16 steps of a few rows hand the
    # norms from product to product (the final one to the head where every row's logits are wanted, the first one from the kernel
    # that fetches the token rows in steps of single tokens): only the first norm of the prompt's step is a kernel
    if dtype == "float32":
        assert int(rows["rmsnorm"][0]) == 2 * layers * steps + steps - 1
    else:
        assert int(rows["rmsnorm"][0]) == 1 and int(rows["embed_handing"][0]) == steps - 1 and int(rows["embed"][0]) == 1
    assert "host work, uploads, downloads" in rows
    shares = [float(v[-1 if len(v) == 3 else -2].rstrip("%")) for k, v in rows.items() if k != "host work, uploads, downloads"]
    assert 0 < sum(shares) <= 100.5
    assert llm.runner.can_step_from_device and not ops.profiling()
    assert llm.generate(prompt, steps=len(prompt) + 5, temperature=0.0).generated_tokens == plain_run
    assert len(llm.runner._graphs) == graphs and llm.profile_report() == ""


def test_temperature_sampling_follows_the_seeded_stream(folders):
    """Tiny B: temperature 0.8 with a seeded generator; every draw is re-derived from the plain
    logits and the plain sampler with the same uniform numbers."""
    import geneinfer_amd as gi
    plain = PlainLlama(folders["B"])
    llm = gi.LLM(folders["B"], dtype="float32", page_size=PAGE_SIZE["B"], max_tokens=128, max_running=2)
    for i, prompt in enumerate(prompts_for("B", [1, 9, 33, 40])):
        got = llm.generate(prompt, steps=len(prompt) + 11, temperature=0.8, seed=70 + i).generated_tokens
        assert len(got) == 12
        us = plain_sampler.uniforms(70 + i, 12)
        toks = list(prompt)
        for step, tok in enumerate(got):
            row = plain.logits(toks)[-1].float().numpy()
            want = plain_sampler.sample(row, 0.8, 0, 1.0, us[step])
            if tok != want:            # a draw on the edge between two tokens may fall either way in 32-bit; nothing else may
                p = torch.softmax(torch.from_numpy(row).double() / 0.8, 0)
                cum = torch.cumsum(p, 0)
                assert abs(tok - want) == 1 and float((cum - float(us[step])).abs().min()) < 1e-5
            toks.append(tok)
    for k, p, seed in ((5, 0.9, 3), (0, 0.7, 4), (3, 1.0, 5)):        # with filters: the same, the order of nearly equal tokens aside
        prompt = prompts_for("B", [9])[0]
        top = llm.generate(prompt, steps=20, temperature=0.8, top_k=k, top_p=p, seed=seed).generated_tokens
        assert len(top) == 12
        us = plain_sampler.uniforms(seed, 12)
        toks = list(prompt)
        for step, tok in enumerate(top):
            row = plain.logits(toks)[-1].float().numpy()
            want = plain_sampler.sample(row, 0.8, k, p, us[step])
            if tok != want:
                near = {plain_sampler.sample(row, 0.8, k, min(max(p + dp, 1e-6), 1.0 - 1e-7) if p < 1.0 else p, min(max(float(us[step]) + du, 0.0), 1.0 - 2.0 ** -24))
                        for dp in (-1e-5, 0.0, 1e-5) for du in (-1e-5, 0.0, 1e-5)}
                assert tok in near, (k, p, step, tok, want)
            toks.append(tok)


@pytest.mark.parametrize("name,temperature", [("A", 0.0), ("B", 0.8)])
def test_scheduler_gives_each_request_what_it_gets_alone(folders, name, temperature):
    """Through the scheduler with few pages (requests are preempted and fed again) every request
    ends with the tokens of the single-request loop, in 32-bit bit for bit."""
    import geneinfer_amd as gi
    from geneinfer_amd.engine import EngineConfig, EngineRequest
    from geneinfer_amd.sampling import SamplerConfig
    lengths = [5, 11, 17, 3, 26, 9] if name == "A" else [1, 9, 33, 40, 12]
    prompts = prompts_for(name, lengths)
    new = 8 if name == "A" else 12
    ps = PAGE_SIZE[name]
    roomy = gi.LLM(folders[name], dtype="float32", page_size=ps, max_tokens=256, max_running=1)
    alone = [roomy.generate(p, steps=len(p) + new - 1, temperature=temperature, seed=5 + i).generated_tokens for i, p in enumerate(prompts)]
    assert all(len(a) == new for a in alone)
    preempted = 0
    tight, tighter = (48, 36) if name == "A" else (96, 56)
    for max_tokens, cfg in ((512, EngineConfig(max_running=4)), (tight, EngineConfig(max_running=4, step_rows=16, prefill_chunk=5)),
                            (tighter, EngineConfig(max_running=3, step_rows=8))):
        llm = gi.LLM(folders[name], dtype="float32", page_size=ps, max_tokens=max_tokens, max_running=4, max_rows=64)
        eng = llm.engine(cfg)
        ids = [eng.submit(EngineRequest(p, len(p) + new - 1, SamplerConfig(temperature, seed=5 + i))) for i, p in enumerate(prompts)]
        eng.run_until_idle()
        for jid, want in zip(ids, alone):
            r = eng.result(jid)
            assert r.finished and r.error == "" and r.generated_tokens == want, (max_tokens, jid, r.preemptions)
        llm.runner.cache.check_consistency()
        if eng.prefix is not None:
            eng.prefix.clear()
        assert llm.runner.cache.free_pages() == [max_tokens // ps]
        preempted += eng.stats.preemptions
    assert preempted > 0, "no pool was tight enough to preempt"


@pytest.mark.parametrize("temperature", [0.0, 0.8])
def test_decoding_ahead_changes_no_token(folders, temperature):
    """The scheduler queues a decode step before it has read the tokens of the last one.  With end tokens that cut
    requests short at different times (a row too many is then computed for them), with requests that wait for a free
    place and with a pool so small that pages run out, every request ends as it does when every step's tokens are read
    first, and as it does alone; and steps were in fact queued ahead."""
    import geneinfer_amd as gi
    from geneinfer_amd.engine import EngineConfig, EngineRequest
    from geneinfer_amd.sampling import SamplerConfig
    name, new, ps = "B", 40, PAGE_SIZE["B"]
    prompts = prompts_for(name, [7, 19, 3, 30, 12, 5], seed=77)
    roomy = gi.LLM(folders[name], dtype="float32", page_size=ps, max_tokens=512, max_running=1)
    free_run = [roomy.generate(p, steps=len(p) + new - 1, temperature=temperature, seed=3 + i).generated_tokens for i, p in enumerate(prompts)]
    end_tokens = {free_run[0][9], free_run[1][23], free_run[3][4]}                  # three requests stop early, at different steps
    roomy.end_tokens = sorted(end_tokens)
    alone = [roomy.generate(p, steps=len(p) + new - 1, temperature=temperature, seed=3 + i) for i, p in enumerate(prompts)]
    assert sum(a.stopped_by_end_token for a in alone) >= 3 and any(not a.stopped_by_end_token for a in alone)
    outcomes = {}
    for ahead in (True, False):
        for max_tokens, max_running in ((1024, 4), (1024, 6), (80, 4)):
            llm = gi.LLM(folders[name], dtype="float32", page_size=ps, max_tokens=max_tokens, max_running=max_running, max_rows=64,
                         end_tokens=sorted(end_tokens))
            eng = llm.engine(EngineConfig(max_running=max_running, decode_ahead=ahead))
            assert (eng._landing_strips is not None) == ahead
            flights = 0
            ids = [eng.submit(EngineRequest(p, len(p) + new - 1, SamplerConfig(temperature, seed=3 + i))) for i, p in enumerate(prompts)]
            while eng.step():
                flights += eng._flight is not None
            assert eng.idle()
            results = [eng.result(j) for j in ids]
            for r, a in zip(results, alone):
                assert r.finished and r.error == "" and r.generated_tokens == a.generated_tokens and r.stopped_by_end_token == a.stopped_by_end_token
            llm.runner.cache.check_consistency()
            if eng.prefix is not None:
                eng.prefix.clear()
            assert llm.runner.cache.free_pages() == [max_tokens // ps]
            assert (flights > 10) == ahead
            outcomes[(ahead, max_tokens, max_running)] = eng.stats
    assert outcomes[(True, 80, 4)].preemptions > 0 and outcomes[(False, 80, 4)].preemptions > 0, "the small pool never ran out"
    # a row too many for each request that an end token stopped while a step was queued ahead, nothing else
    assert 0 <= outcomes[(True, 1024, 6)].rows - outcomes[(False, 1024, 6)].rows <= sum(a.stopped_by_end_token for a in alone)


def test_samplers_of_every_kind_side_by_side(folders):
    """Greedy, plain and filtering (top-k, top-p, both) requests in one engine, their decode steps queued ahead: each ends
    with the tokens it gets alone, and a filtering request alone decodes ahead as well."""
    import geneinfer_amd as gi
    from geneinfer_amd.engine import EngineConfig, EngineRequest
    from geneinfer_amd.sampling import SamplerConfig
    name, new, ps = "B", 24, PAGE_SIZE["B"]
    prompts = prompts_for(name, [7, 19, 3, 30, 12, 5], seed=78)
    samplers = [SamplerConfig(0.0), SamplerConfig(0.8, seed=11), SamplerConfig(0.9, top_k=6, seed=12), SamplerConfig(1.1, top_p=0.6, seed=13),
                SamplerConfig(0.7, top_k=12, top_p=0.8, seed=14), SamplerConfig(0.0)]
    roomy = gi.LLM(folders[name], dtype="float32", page_size=ps, max_tokens=512, max_running=1)
    alone = [roomy.generate(p, steps=len(p) + new - 1, temperature=c.temperature, top_k=c.top_k, top_p=c.top_p, seed=c.seed).generated_tokens
             for p, c in zip(prompts, samplers)]
    assert all(len(a) == new for a in alone) and len({tuple(a) for a in alone}) == len(alone)
    for max_running in (6, 3):
        llm = gi.LLM(folders[name], dtype="float32", page_size=ps, max_tokens=1024, max_running=max_running, max_rows=64)
        eng = llm.engine(EngineConfig(max_running=max_running))
        ids = [eng.submit(EngineRequest(p, len(p) + new - 1, c)) for p, c in zip(prompts, samplers)]
        flights = 0
        while eng.step():
            flights += eng._flight is not None
        assert flights > 10
        for j, want in zip(ids, alone):
            assert eng.result(j).generated_tokens == want, (max_running, j)
    llm = gi.LLM(folders[name], dtype="float32", page_size=ps, max_tokens=512, max_running=2, max_rows=64)
    eng = llm.engine(EngineConfig(max_running=2))
    ids = [eng.submit(EngineRequest(prompts[i], len(prompts[i]) + new - 1, samplers[i])) for i in (2, 4)]
    flights = 0
    while eng.step():
        flights += eng._flight is not None
    assert flights > 10 and [eng.result(j).generated_tokens for j in ids] == [alone[2], alone[4]]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_requests_with_an_equal_beginning_share_its_pages(folders, dtype):
    """Requests that begin alike take the pages an earlier one computed: fewer rows are fed, and every request still
    ends with the tokens it gets alone (bit for bit in 32-bit, where the keys of a position never depend on the batch)."""
    import geneinfer_amd as gi
    from geneinfer_amd.engine import EngineConfig, EngineRequest, StepEntry
    from geneinfer_amd.sampling import SamplerConfig
    name, new = "B", 10
    system = prompts_for(name, [70], seed=31)[0]
    tails = prompts_for(name, [5, 1, 12, 30], seed=32)
    prompts = [system + t for t in tails] + [system[:40], tails[3] + system]
    def run(prefix_cache, max_tokens, watch=False):
        from geneinfer_amd.engine import Engine
        from geneinfer_amd.sampling import sample_rows
        llm = gi.LLM(folders[name], dtype=dtype, page_size=16, max_tokens=max_tokens, max_running=3, max_rows=64)
        seen = []                                                    # (sampler, logits row) of every draw, when watched (no step is then queued ahead)
        def watching(logits, samplers):
            seen.extend(zip(samplers, logits.cpu()))
            return sample_rows(logits, samplers)
        cfg = EngineConfig(max_running=3, step_rows=48, prefix_cache=prefix_cache)
        eng = Engine(llm.runner, cfg, llm.end_tokens, sample=watching) if watch else llm.engine(cfg)
        ids = [eng.submit(EngineRequest(prompts[0], len(prompts[0]) + new - 1, SamplerConfig(0.0)))]
        eng.run_until_idle()                                         # the first one has finished when the others arrive
        ids += [eng.submit(EngineRequest(p, len(p) + new - 1, SamplerConfig(0.0))) for p in prompts[1:]]
        eng.run_until_idle()
        llm.runner.cache.check_consistency()
        by_sampler = {}
        for sampler, row in seen:
            by_sampler.setdefault(id(sampler), []).append(row)
        return llm, eng, [eng.result(j) for j in ids], [by_sampler.get(id(eng.jobs[j].sampler), []) for j in ids]
    _, plain_eng, plain, _ = run(False, 1024)
    exact, rounded = PlainLlama(folders[name]), PlainLlama(folders[name], storage=torch.bfloat16)

    def compare(got, want, near, what):
        if dtype == "float32":
            worst = max(relative_error(row, want[key]) for key, row in got.items())
            assert worst < 2e-5, (what, worst)
        else:
            assert_within_bfloat16_noise(got, want.__getitem__, near.__getitem__, what)

    # roomy; so tight that named pages must be given back; and tight again with the logits of every draw watched
    for max_tokens, watch in ((1024, False), (192, False), (192, True)):
        llm, eng, shared, drawn_from = run(True, max_tokens, watch)
        assert eng.prefix is not None and eng.stats.prefix_hits >= 4 and eng.stats.prefix_tokens >= 3 * 64 + 32
        assert eng.stats.rows <= plain_eng.stats.rows - (3 * 64 + 32) + 64 * eng.stats.preemptions
        for a, b in zip(shared, plain):
            assert a.finished and a.error == "" and len(a.generated_tokens) == len(b.generated_tokens)
            if dtype == "float32":
                assert a.generated_tokens == b.generated_tokens
        assert sum(r.cached_tokens for r in shared) == eng.stats.prefix_tokens
        if max_tokens == 192:
            assert eng.stats.evicted_pages > 0 or eng.stats.preemptions > 0
        if watch:
            # Every token was drawn from the plain model's logits for the request's tokens so far, whichever pages were shared,
            # given back and computed again on the way (a request fed again after a preemption draws its next new token only).
            got, want, near = {}, {}, {}
            for i, (r, rows) in enumerate(zip(shared, drawn_from)):
                tokens = prompts[i] + r.generated_tokens
                assert len(rows) == len(r.generated_tokens) == new
                e, nr = exact.logits(tokens[:-1]), rounded.logits(tokens[:-1])
                for k, row in enumerate(rows):
                    at = len(prompts[i]) - 1 + k
                    got[(i, k)], want[(i, k)], near[(i, k)] = row, e[at], nr[at]
                    assert int(torch.argmax(row)) == r.generated_tokens[k]
            compare(got, want, near, f"draws behind shared pages, pool of {max_tokens}")
        # What the shared pages hold, in either precision: every prompt again, opened on the pages the index still names for
        # it, the rest fed in one step; the logits behind the shared pages are the plain model's for the whole prompt.
        runner, index, got, want, near, found = llm.runner, llm.runner.cache.prefix, {}, {}, {}, 0
        for i, prompt in enumerate(prompts):
            pages = index.match(prompt, len(prompt) - 1)
            found += len(pages)
            if i != 5 and max_tokens == 1024:
                assert len(pages) >= (2 if i == 4 else 4)            # 70 equal tokens are four full pages of 16, 40 are two
            runner.open(("again", i), pages)
            held = runner.length(("again", i))
            rows = runner.step([StepEntry(("again", i), prompt[held:], tuple(range(len(prompt) - held)))]).cpu()
            runner.close(("again", i))
            e, r = exact.logits(prompt), rounded.logits(prompt)
            for k, row in enumerate(rows):
                got[(i, held + k)], want[(i, held + k)], near[(i, held + k)] = row, e[held + k], r[held + k]
        assert found >= 4, "the index names no page of the prompts it has just served"
        compare(got, want, near, f"rows behind shared pages, pool of {max_tokens}")
        runner.cache.check_consistency()


def test_scheduler_in_bfloat16_runs_mixed_batches(folders):
    """Through the scheduler in bfloat16 (portions of prompts beside decoding requests, four at a time): the logits every
    token is drawn from are the plain model's for the request's tokens so far, within what rounding explains."""
    import geneinfer_amd as gi
    from geneinfer_amd.engine import Engine, EngineConfig, EngineRequest
    from geneinfer_amd.sampling import SamplerConfig, sample_rows
    llm = gi.LLM(folders["B"], dtype="bfloat16", page_size=16, max_tokens=512, max_running=4, max_rows=64)
    prompts = prompts_for("B", [1, 9, 33, 40, 12, 70])
    seen = []                                                         # (sampler, logits row) of every draw
    def watching(logits, samplers):
        seen.extend(zip(samplers, logits.cpu()))
        return sample_rows(logits, samplers)
    eng = Engine(llm.runner, EngineConfig(max_running=4, step_rows=24), llm.end_tokens, sample=watching)
    ids = [eng.submit(EngineRequest(p, 90, SamplerConfig(0.0))) for p in prompts]
    eng.run_until_idle()
    out = [eng.result(i) for i in ids]
    assert all(r.finished and r.error == "" and len(r.generated_tokens) == 90 - len(p) + 1 for r, p in zip(out, prompts))
    assert eng.stats.max_rows_in_pass > 4 and eng.stats.max_running_seen == 4
    exact, rounded = PlainLlama(folders["B"]), PlainLlama(folders["B"], storage=torch.bfloat16)
    by_sampler = {}
    for sampler, row in seen:
        by_sampler.setdefault(id(sampler), []).append(row)
    got, want, near = {}, {}, {}
    for n, (r, p) in enumerate(zip(out, prompts)):
        rows = by_sampler[id(eng.jobs[ids[n]].sampler)]
        tokens = p + r.generated_tokens
        assert len(rows) == len(r.generated_tokens)
        e, nr = exact.logits(tokens[:-1]), rounded.logits(tokens[:-1])
        for k, row in enumerate(rows):                                 # draw k saw the logits at position len(p) - 1 + k
            got[(n, k)], want[(n, k)], near[(n, k)] = row, e[len(p) - 1 + k], nr[len(p) - 1 + k]
            assert int(torch.argmax(row)) == r.generated_tokens[k]
    assert_within_bfloat16_noise(got, want.__getitem__, near.__getitem__, "scheduler in bfloat16")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(folders, dtype):
    """300 tokens, all but the first 10 fed one by one (decode steps replay a captured graph from
    the second on): the logits still equal the plain model's over the whole sequence.

    32-bit: against the 64-bit plain model, 2e-5.  bfloat16: within the rounding noise."""
    from geneinfer_amd.engine import Runner, StepEntry, load_model
    toks = prompts_for("B", [300], seed=21)[0]
    model = load_model(folders["B"], dtype, "cuda:0")
    runner = Runner(model, page_size=16, max_tokens=320, max_requests=2)
    runner.open("r")
    runner.step([StepEntry("r", toks[:10], ())])
    got = {}
    for p in range(10, 300):
        got[p] = runner.step([StepEntry("r", [toks[p]], (0,))])[0].cpu()
    exact = PlainLlama(folders["B"]).logits(toks)
    if dtype == "float32":
        worst = max(relative_error(row, exact[p]) for p, row in got.items())
        assert worst < 2e-5, worst
    else:
        rounded = PlainLlama(folders["B"], storage=torch.bfloat16).logits(toks)
        assert_within_bfloat16_noise(got, lambda p: exact[p], lambda p: rounded[p], "long decoding")
    assert runner._graphs and all(g.graph is not None for g in runner._graphs.values()), "decode steps did not replay a graph"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_graphs_across_a_context_bracket_and_between_batch_sizes(folders, dtype):
    """Captured decode steps are kept per (batch size, power-of-two bracket of the longest context from 1024 on), and the
    bracket fixes how the attention kernel cuts contexts into pieces.  Three requests decode with the longest crossing
    position 1024 -> 1025 meanwhile (one stays short, far on the other side of the bracket), in steps of three and of two
    requests by turns, so that four graphs are captured and each is replayed after another one: every logit row is the
    plain model's.  Then a runner that may keep two graphs only does the same."""
    from geneinfer_amd.engine import Runner, StepEntry, load_model
    seqs = dict(zip("abc", prompts_for("D", [1060, 1050, 90], seed=17)))
    start = {"a": 1000, "b": 990, "c": 30}
    model = load_model(folders["D"], dtype, "cuda:0")
    exact, rounded = PlainLlama(folders["D"]), PlainLlama(folders["D"], storage=torch.bfloat16)
    want = {r: exact.logits(t) for r, t in seqs.items()}
    near = {r: rounded.logits(t) for r, t in seqs.items()} if dtype == "bfloat16" else None
    for max_graphs in (16, 2):
        runner = Runner(model, page_size=16, max_tokens=2304, max_requests=3, max_graphs=max_graphs)
        for r, t in seqs.items():
            runner.open(r)
            runner.step([StepEntry(r, t[:start[r]], ())])
        got, at = {}, dict(start)
        for k in range(60):
            batch = ["a", "b", "c"] if k % 2 == 0 else ["a", "b"]
            logits = runner.step([StepEntry(r, [seqs[r][at[r]]], (0,)) for r in batch]).cpu()
            for r, row in zip(batch, logits):
                got[(r, at[r])] = row
                at[r] += 1
        assert at == {"a": 1060, "b": 1050, "c": 60}
        if max_graphs == 16:
            assert set(runner._graphs) == {(3, 1024), (2, 1024), (3, 2048), (2, 2048)} and all(g.graph is not None and g.calls >= 4 for g in runner._graphs.values())
        else:
            assert len(runner._graphs) == 2
        if dtype == "float32":
            worst = max(relative_error(row, want[r][p]) for (r, p), row in got.items())
            assert worst < 2e-5, worst
        else:
            assert_within_bfloat16_noise(got, lambda k: want[k[0]][k[1]], lambda k: near[k[0]][k[1]], f"graphs across brackets, {max_graphs} kept")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decode_steps_filled_up_to_a_captured_batch_size(folders, dtype):
    """Above 8 requests a decode step runs at the next batch size of a short list, filled up with rows of the spare slot.  Eleven
    requests decode, finish one after the other down to nine, and go on: the steps of 11 and 12 requests share one graph,
    those of 9 and 10 another; every logit row is the plain model's (in 32-bit also bit for bit what a runner without graphs
    gives), and the rows that filled the steps up have touched no request's page: the pool is whole at the end."""
    from geneinfer_amd.engine import Runner, StepEntry, load_model
    n_requests, new = 11, 14
    seqs = {f"r{i}": t for i, t in enumerate(prompts_for("B", [20 + 3 * i for i in range(n_requests)], seed=23))}
    model = load_model(folders["B"], dtype, "cuda:0")
    exact, rounded = PlainLlama(folders["B"]), PlainLlama(folders["B"], storage=torch.bfloat16)
    want = {r: exact.logits(t) for r, t in seqs.items()}
    near = {r: rounded.logits(t) for r, t in seqs.items()} if dtype == "bfloat16" else None
    runs = {}
    for use_graphs in (True, False):
        runner = Runner(model, page_size=8, max_tokens=n_requests * 64, max_requests=n_requests, use_graphs=use_graphs)
        start = {r: len(t) - new for r, t in seqs.items()}
        for r, t in seqs.items():
            runner.open(r)
            runner.step([StepEntry(r, t[:start[r]], ())])
        got, at, live = {}, dict(start), list(seqs)
        for k in range(new):
            if k in (5, 9):                            # 11 -> 10 -> 9 requests
                runner.close(live.pop(3))
            logits = runner.step([StepEntry(r, [seqs[r][at[r]]], (0,)) for r in live]).cpu()
            assert logits.shape[0] == len(live)
            for r, row in zip(live, logits):
                got[(r, at[r])] = row
                at[r] += 1
        if use_graphs:
            assert set(runner._graphs) == {(12, 1024), (10, 1024)}, set(runner._graphs)
            assert all(g.graph is not None for g in runner._graphs.values())
        for r in live:
            runner.close(r)
        runner.cache.check_consistency()
        assert runner.cache.free_pages() == [g.pool.n_pages for g in runner.cache.groups]
        runs[use_graphs] = got
    got = runs[True]
    if dtype == "float32":
        worst = max(relative_error(row, want[r][p]) for (r, p), row in got.items())
        assert worst < 2e-5, worst
        assert all(torch.equal(row, runs[False][key]) for key, row in got.items())
    else:
        assert_within_bfloat16_noise(got, lambda k: want[k[0]][k[1]], lambda k: near[k[0]][k[1]], "filled-up decode steps")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_pages_far_into_a_large_cache(folders, dtype):
    """A cache of more than 2^31 elements a layer: with the low pages taken, two requests live in pages whose offsets need
    more than 32 bits (in elements and in bytes), a prompt in portions and single tokens beside it.  Every kernel that
    touches the cache (rotation and page write, prompt and decode attention, the fused decode step) meets them."""
    from geneinfer_amd.engine import Runner, StepEntry, load_model
    model = load_model(folders["D"], dtype, "cuda:0")
    per_page = 2 * CONFIGS["D"]["num_key_value_heads"] * 16 * 64                    # elements of a page in one layer
    n_pages = (1 << 31) // per_page + 200
    runner = Runner(model, page_size=16, max_tokens=16 * n_pages, max_requests=2)
    pool = runner.cache.groups[0].pool
    held = [pool.allocate() for _ in range(n_pages - 150)]                          # what is left lies beyond 2^31 elements
    assert min(pool._free) * per_page > (1 << 31)
    seqs = dict(zip("ab", prompts_for("D", [700, 330], seed=29)))
    exact, rounded = PlainLlama(folders["D"]), PlainLlama(folders["D"], storage=torch.bfloat16)
    want = {r: exact.logits(t) for r, t in seqs.items()}
    near = {r: rounded.logits(t) for r, t in seqs.items()} if dtype == "bfloat16" else None
    got = {}
    def run(entries):
        logits = runner.step([StepEntry(r, seqs[r][a:b], tuple(range(b - a))) for r, a, b in entries]).cpu()
        rows = iter(logits)
        for r, a, b in entries:
            for p in range(a, b):
                got[(r, p)] = next(rows)
    runner.open("a"); runner.open("b")
    run([("a", 0, 300)])
    run([("a", 300, 640), ("b", 0, 290)])
    for k in range(40):                                                             # a: 640..679 singly, b: 290..329 singly, captured from the second step on
        run([("a", 640 + k, 641 + k), ("b", 290 + k, 291 + k)])
    run([("a", 680, 700)])
    assert int(min(runner.cache.page_row("a"))) * per_page > (1 << 31)
    if dtype == "float32":
        worst = max(relative_error(row, want[r][p]) for (r, p), row in got.items())
        assert worst < 2e-5, worst
    else:
        assert_within_bfloat16_noise(got, lambda k: want[k[0]][k[1]], lambda k: near[k[0]][k[1]], "pages far into a large cache")
    runner.close("a"); runner.close("b")
    for page in held:
        pool.release(page)
    runner.cache.check_consistency()
    del runner
    torch.cuda.empty_cache()


@pytest.mark.parametrize("dtype,tol", [("float32", 2e-5), ("bfloat16", 1.5e-2)])
def test_first_tokens_of_a_sequence(folders, dtype, tol):
    """Positions 0, 1, 2: one key, two keys; a prompt of one token; a page edge at position 4."""
    from geneinfer_amd.engine import Runner, StepEntry, load_model
    model = load_model(folders["A"], dtype, "cuda:0")
    plain = PlainLlama(folders["A"], storage=torch.bfloat16 if dtype == "bfloat16" else None)
    toks = prompts_for("A", [6], seed=2)[0]
    want = plain.logits(toks)
    for cut in ([1, 1, 1, 1, 1, 1], [1, 5], [2, 1, 3], [6]):
        runner = Runner(model, page_size=16 if dtype == "bfloat16" else 4, max_tokens=64, max_requests=2)
        runner.open("r")
        p = 0
        for n in cut:
            logits = runner.step([StepEntry("r", toks[p:p + n], tuple(range(n)))])
            for i in range(n):
                assert relative_error(logits[i], want[p + i]) < tol, (cut, p + i)
            p += n


def test_step_refuses_bad_batches_and_changes_nothing(folders):
    from geneinfer_amd.cache import OutOfPages
    from geneinfer_amd.engine import Runner, StepEntry, StepError, load_model
    model = load_model(folders["A"], "float32", "cuda:0")
    runner = Runner(model, page_size=4, max_tokens=16, max_requests=2, max_rows=16, max_positions=12)
    runner.open("a"); runner.open("b")
    runner.step([StepEntry("a", [1, 2, 3], ())])
    for bad, msg in (([], "at least one entry"), ([StepEntry("zz", [1])], "not open"), ([StepEntry("a", [])], "no tokens"),
                     ([StepEntry("a", [256])], "outside the vocabulary"), ([StepEntry("a", [1], (1,))], "wants logits at place 1"),
                     ([StepEntry("a", [1]), StepEntry("a", [2])], "twice"), ([StepEntry("a", [1] * 10)], "position limit 12"),
                     ([StepEntry("a", [1] * 8), StepEntry("b", [1] * 9)], "max_rows"),
                     # a caller that names the position of its first token is held to what the cache holds
                     ([StepEntry("a", [1], (0,), at=4)], "leaves a gap: the cache holds 3"), ([StepEntry("a", [1, 2], at=2)], "lies under the 3 positions"),
                     ([StepEntry("a", [1], at=-1)], "exceed the context length 12"), ([StepEntry("b", [1] * 4, at=9)], "exceed the context length 12"),
                     ([StepEntry("b", [1], (0,), at=1)], "leaves a gap: the cache holds 0")):
        with pytest.raises(StepError, match=msg):
            runner.step(bad)
    assert runner.length("a") == 3 and runner.length("b") == 0
    named = runner.step([StepEntry("b", [9], (0,), at=0)])             # the right position changes nothing
    runner.truncate("b", 0)
    assert torch.equal(named, runner.step([StepEntry("b", [9], (0,))]))
    runner.truncate("b", 0)
    with pytest.raises(OutOfPages):                                   # 4 pages in all: a holds 1 and needs 2 more, b needs 2
        runner.step([StepEntry("a", [5] * 8, ()), StepEntry("b", [5] * 8, ())])
    assert runner.length("a") == 3 and runner.length("b") == 0 and runner.cache.free_pages() == [3]
    last = runner.step([StepEntry("a", [7] * 9, (8,))])               # the exact last position is allowed
    assert last.shape == (1, 256) and runner.length("a") == 12
    with pytest.raises(StepError, match="position limit"):
        runner.step([StepEntry("a", [1])])
