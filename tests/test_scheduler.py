"""The scheduler's decisions without a GPU: a stand-in step function over the real cache manager
returns logits that depend on everything a request has been fed, so a request that is cut,
batched, preempted and fed again must still produce the tokens it produces alone."""
import hashlib
import random
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from geneinfer_amd.cache import CacheManager, OutOfPages, PagedKvNeed
from geneinfer_amd.engine import POOL_TOO_SMALL, Engine, EngineConfig, EngineRequest, StepEntry, generate
from geneinfer_amd.sampling import Sampler, SamplerConfig, filtered_draw

VOCAB = 50


class FakeRunner:
    """What the scheduler needs of a runner, with logits = a hash of the request's tokens so far."""

    def __init__(self, page_size=4, n_pages=64, max_requests=8, max_rows=64, max_positions=96, windows=False):
        needs = [PagedKvNeed(1, 2), PagedKvNeed(1, 2, window=12)] if windows else [PagedKvNeed(1, 2)]
        self.cache = CacheManager(needs, [None] * len(needs), page_size=page_size, n_pages=n_pages, max_requests=max_requests,
                                  max_positions=max_positions, allocate_storage=False)
        self.model = SimpleNamespace(spec=SimpleNamespace(vocab_size=VOCAB))
        self.max_rows, self.max_positions = max_rows, max_positions
        self.fed, self.log = {}, []
        self.page_size, self.on_page = page_size, {}          # what each page of the first group holds, place by place

    def open(self, r, shared_pages=()):
        self.cache.open(r, shared_pages)
        self.fed[r] = [self.on_page[(int(p), i)] for p in shared_pages for i in range(self.page_size)]      # what the shared pages hold

    def close(self, r):
        self.cache.close(r)
        del self.fed[r]

    def is_open(self, r):
        return self.cache.is_open(r)

    def step(self, entries):
        assert 0 < sum(len(e.tokens) for e in entries) <= self.max_rows
        self.cache.reserve([(e.request, len(e.tokens)) for e in entries])
        rows = []
        for e in entries:
            assert len(self.fed[e.request]) == self.cache.length(e.request)
            for i, t in enumerate(e.tokens):
                at = len(self.fed[e.request])
                page = self.cache.pages_of(e.request)[at // self.page_size - int(self.cache.groups[0].first_live[self.cache.slot(e.request)])]
                assert self.cache.groups[0].pool.ref_count(page) == 1 or (self.cache.prefix is not None and page in self.cache.prefix and
                                                                          self.cache.groups[0].pool.ref_count(page) == 2 and False), "a shared page is written"
                self.on_page[(page, at % self.page_size)] = int(t)
                self.fed[e.request].append(int(t))
                if i in e.want:
                    seed = int.from_bytes(hashlib.sha256(str(self.fed[e.request]).encode()).digest()[:8], "little")
                    rows.append(np.random.default_rng(seed).standard_normal(VOCAB).astype(np.float32) * 2)
            self.cache.advance(e.request, len(e.tokens))
        self.log.append([(e.request, len(e.tokens), tuple(e.want)) for e in entries])
        self.cache.check_consistency()
        return torch.from_numpy(np.stack(rows)) if rows else None


def pages_when_forgotten(runner):
    """Free pages per group once the prefix index has let go of what it keeps."""
    runner.cache.check_consistency()
    if runner.cache.prefix is not None:
        assert runner.cache.prefix.evictable() == len(runner.cache.prefix)       # nobody else holds them
        runner.cache.prefix.clear()
    return runner.cache.free_pages()


def host_sample_row(row, sampler):
    if sampler.config.greedy:
        return int(np.argmax(row.numpy()))
    return filtered_draw(row.numpy(), sampler.config, sampler.next_uniform())


def host_sample(logits, samplers):
    return [host_sample_row(row, s) for row, s in zip(logits, samplers)]


def alone(prompt, max_positions, cfg, end_tokens):
    r = generate(FakeRunner(n_pages=64), Sampler(cfg, VOCAB), prompt, max_positions, end_tokens, sample=host_sample_row)
    return r.generated_tokens, r.stopped_by_end_token


def make_requests(rng, n):
    out = []
    for i in range(n):
        prompt = [rng.randrange(VOCAB) for _ in range(rng.choice([1, 2, 5, 9, 17, 30]))]
        limit = rng.choice([0, len(prompt) + rng.randint(1, 25), max(1, len(prompt) - 2)])
        cfg = SamplerConfig(temperature=rng.choice([0.0, 0.8, 1.3]), top_k=rng.choice([0, 5]), top_p=rng.choice([1.0, 0.9]), seed=100 + i)
        out.append((prompt, limit, cfg))
    return out


END = {7, 31}                                     # about one token in 25 ends a request


@pytest.mark.parametrize("n_pages,max_running,step_rows,chunk", [
    (64, 4, 0, 0), (64, 1, 0, 0), (64, 6, 1, 0), (64, 3, 3, 1), (40, 4, 8, 5), (30, 4, 64, 16), (26, 5, 8, 0), (25, 3, 3, 5),
    (25, 6, 64, 0), (48, 2, 5, 16), (24, 8, 0, 0), (24, 4, 8, 3),
])
@pytest.mark.parametrize("prefix_cache", [False, True])
def test_every_request_gets_the_tokens_it_gets_alone(n_pages, max_running, step_rows, chunk, prefix_cache):      # src/runtime/engine.h:8-9, tools/engine_check_main.cpp:179-211
    rng = random.Random(n_pages * 100 + max_running)
    requests = make_requests(rng, 9)
    if prefix_cache:                                                   # some requests start like others, by one page and more
        requests[3] = (requests[2][0][:9] + requests[3][0], *requests[3][1:])
        requests[6] = (requests[2][0] + requests[6][0], 0, requests[6][2])
        requests[7] = (list(requests[6][0]), 0, requests[7][2])
    runner = FakeRunner(n_pages=n_pages, max_requests=8, max_rows=64)
    eng = Engine(runner, EngineConfig(max_running, step_rows, chunk, prefix_cache), END, sample=host_sample)
    assert (eng.prefix is not None) == prefix_cache
    ids = [eng.submit(EngineRequest(p, limit, cfg)) for p, limit, cfg in requests[:5]]
    for _ in range(3):                                                 # the rest arrive while the first are running
        eng.step()
    ids += [eng.submit(EngineRequest(p, limit, cfg)) for p, limit, cfg in requests[5:]]
    eng.run_until_idle()
    assert eng.idle() and not runner.cache.open_requests()
    runner.cache.check_consistency()
    if prefix_cache:                                                   # what is not free is what the prefix index keeps
        assert runner.cache.free_pages() == [n_pages - len(eng.prefix)] and eng.prefix.evictable() == len(eng.prefix)
        eng.prefix.clear()
    assert runner.cache.free_pages() == [n_pages]                      # nothing leaked
    for jid, (prompt, limit, cfg) in zip(ids, requests):
        res = eng.result(jid)
        want_tokens, want_end = alone(prompt, limit, cfg, END)
        assert res.finished and res.error == ""
        assert (res.generated_tokens, res.stopped_by_end_token) == (want_tokens, want_end), (jid, res.preemptions)
    rows_limit = min(step_rows or 64, 64)
    for entries in runner.log:
        assert sum(n for _, n, _ in entries) <= rows_limit and len(entries) <= min(max_running, 8)
        if chunk:
            assert all(n <= chunk for _, n, _ in entries)
    st = eng.stats
    assert st.passes == len(runner.log) and st.rows == sum(n for e in runner.log for _, n, _ in e)
    assert st.max_rows_in_pass <= rows_limit and st.max_running_seen <= max_running
    assert st.prefix_tokens == sum(eng.result(j).cached_tokens for j in ids) and (st.prefix_hits > 0) == (st.prefix_tokens > 0)
    assert prefix_cache or st.prefix_tokens == 0
    print(f"pages {n_pages}: {st.passes} passes, {st.preemptions} preemptions, {st.prefix_hits} prefix hits ({st.prefix_tokens} positions), "
          f"{st.evicted_pages} pages evicted")
    test_every_request_gets_the_tokens_it_gets_alone.preemptions += st.preemptions


test_every_request_gets_the_tokens_it_gets_alone.preemptions = 0


def test_the_sweep_did_preempt():
    """The tight pools above must have forced requests out (tests/verify_engine.py:98-103)."""
    assert test_every_request_gets_the_tokens_it_gets_alone.preemptions > 0


def test_decoding_requests_come_first_then_prompts_oldest_first():
    runner = FakeRunner(n_pages=64, max_rows=16)
    eng = Engine(runner, EngineConfig(max_running=4, step_rows=16, prefill_chunk=6), sample=host_sample)
    a = eng.submit(EngineRequest(list(range(1, 4)), 40, SamplerConfig(0.0)))       # 3 tokens
    eng.step()                                                                     # a: whole prompt, samples
    b = eng.submit(EngineRequest(list(range(1, 21)), 40, SamplerConfig(0.0)))      # 20 tokens
    c = eng.submit(EngineRequest(list(range(5, 15)), 40, SamplerConfig(0.0)))      # 10 tokens
    eng.step()
    assert runner.log[0] == [(("job", a), 3, (2,))]
    assert runner.log[1] == [(("job", a), 1, (0,)), (("job", b), 6, ()), (("job", c), 6, ())]      # decode row first, chunks of 6, oldest first
    eng.step()
    assert runner.log[2] == [(("job", a), 1, (0,)), (("job", b), 6, ()), (("job", c), 4, (3,))]    # c's last prompt token wants logits
    eng.step()
    assert [e[:2] for e in runner.log[3]] == [(("job", a), 1), (("job", c), 1), (("job", b), 6)]   # c decodes now: before b's chunk


def test_the_budget_shortens_the_last_portion():
    runner = FakeRunner(n_pages=64, max_rows=64)
    eng = Engine(runner, EngineConfig(max_running=3, step_rows=10), sample=host_sample)
    for n in (7, 7):
        eng.submit(EngineRequest([1] * n, 30, SamplerConfig(0.0)))
    eng.step()
    assert [n for _, n, _ in runner.log[0]] == [7, 3]


def test_a_portion_cut_by_the_budget_is_cut_at_a_round_number_when_asked():
    """With a quantum a portion that the budget cuts short ends at a multiple of it (the steps of a long prompt then have one
    shape); the prompt's own end is never rounded, and without a quantum the budget is used to the last row."""
    for quantum, want in ((0, [1, 29, 29, 29, 15]), (8, [1, 24, 24, 24, 24, 6])):
        runner = FakeRunner(page_size=4, n_pages=64, max_rows=64, max_positions=200)
        eng = Engine(runner, EngineConfig(max_running=2, step_rows=30, portion_quantum=quantum), sample=host_sample)
        eng.submit(EngineRequest([1], 200, SamplerConfig(0.0)))                    # decodes beside the prompt below
        eng.step()
        eng.submit(EngineRequest([2] * 102, 200, SamplerConfig(0.0)))
        taken = [1]
        while eng.jobs[1].fed < 101:
            eng.step()
            taken.append(runner.log[-1][1][1])
        assert taken == want, (quantum, taken)


def test_portions_shrink_to_the_free_pages_and_the_youngest_is_preempted():
    runner = FakeRunner(page_size=4, n_pages=6, max_rows=64)                       # 24 positions in all
    eng = Engine(runner, EngineConfig(max_running=3), sample=host_sample)
    x = eng.submit(EngineRequest([1] * 10, 24, SamplerConfig(0.0)))
    y = eng.submit(EngineRequest([2] * 18, 22, SamplerConfig(0.0)))
    eng.step()
    assert [n for _, n, _ in runner.log[0]] == [10, 12]                            # y's portion shrank to the 3 pages left
    eng.run_until_idle()
    assert eng.stats.preemptions >= 1 and eng.result(y).preemptions >= 1 and eng.result(x).preemptions == 0      # the youngest goes
    for jid, prompt, limit in ((x, [1] * 10, 24), (y, [2] * 18, 22)):
        assert eng.result(jid).generated_tokens == alone(prompt, limit, SamplerConfig(0.0), ())[0]
    assert pages_when_forgotten(runner) == [6]


def test_a_lone_request_that_cannot_fit_fails_with_the_reference_message():        # src/runtime/engine.cpp:157-163
    runner = FakeRunner(page_size=4, n_pages=3, max_rows=64)
    eng = Engine(runner, sample=host_sample)
    big = eng.submit(EngineRequest([3] * 8, 40, SamplerConfig(0.0)))
    eng.run_until_idle()
    r = eng.result(big)
    assert r.finished and r.error == POOL_TOO_SMALL and len(r.generated_tokens) == 12 - 8 + 1
    assert runner.cache.free_pages()[0] + runner.cache.evictable_pages() == 3
    small = eng.submit(EngineRequest([3] * 5, 9, SamplerConfig(0.0)))              # the engine goes on afterwards
    eng.run_until_idle()
    assert eng.result(small).error == "" and len(eng.result(small).generated_tokens) == 5


def test_end_tokens_and_position_limits():
    runner = FakeRunner()
    prompt = [4, 8, 15, 16, 23, 42]
    free_run, _ = alone(prompt, 40, SamplerConfig(0.0), ())
    stop = free_run[3]
    eng = Engine(runner, end_tokens=[stop], sample=host_sample)
    j = eng.submit(EngineRequest(prompt, 40, SamplerConfig(0.0)))
    k = eng.submit(EngineRequest(prompt, 4, SamplerConfig(0.0)))                   # the limit lies inside the prompt
    seen = []
    m = eng.submit(EngineRequest(prompt, len(prompt) + 2, SamplerConfig(0.0), on_token=seen.append))
    eng.run_until_idle()
    first_stop = free_run.index(stop)
    assert eng.result(j).generated_tokens == free_run[:first_stop + 1] and eng.result(j).stopped_by_end_token
    assert eng.result(k).finished and eng.result(k).generated_tokens == [] and not eng.result(k).stopped_by_end_token
    assert eng.result(m).generated_tokens == free_run[:3] and seen == [t for t in free_run[:3] if t != stop]


def test_submit_refuses_bad_requests():
    eng = Engine(FakeRunner(max_positions=20), sample=host_sample)
    with pytest.raises(ValueError, match="no tokens"):
        eng.submit(EngineRequest([]))
    with pytest.raises(ValueError, match="does not fit in the context length 20"):
        eng.submit(EngineRequest([1] * 21))
    with pytest.raises(ValueError, match="out of range"):
        eng.submit(EngineRequest([1, VOCAB]))
    with pytest.raises(ValueError, match="top_p"):
        eng.submit(EngineRequest([1], sampler=SamplerConfig(top_p=0.0)))
    with pytest.raises(ValueError, match="max_running"):
        Engine(FakeRunner(), EngineConfig(max_running=0))
    with pytest.raises(IndexError):
        eng.result(3)
    assert eng.step() is False                                                     # nothing to do


def test_windowed_groups_are_planned_per_group():
    runner = FakeRunner(page_size=4, n_pages=10, windows=True)                     # the full group fills up, the windowed one never does
    eng = Engine(runner, EngineConfig(max_running=2), sample=host_sample)
    j = eng.submit(EngineRequest([1] * 12, 36, SamplerConfig(0.0)))
    eng.run_until_idle()
    assert eng.result(j).error == "" and len(eng.result(j).generated_tokens) == 25
    assert runner.cache.free_pages() == [10, 10]


def test_requests_with_an_equal_beginning_share_its_pages():                       # src/runtime/engine.cpp:64-98
    runner = FakeRunner(page_size=4, n_pages=32, max_rows=64)
    eng = Engine(runner, EngineConfig(max_running=1), sample=host_sample)          # one after the other
    system = [rng_token for rng_token in range(10, 23)]                            # 13 tokens: 3 full pages and one more
    prompts = [system + [1, 2], system + [3], system[:8], system[:9], [9] + system]
    limits = [20, 0, 9, 0, 0]
    ids = [eng.submit(EngineRequest(p, lim, SamplerConfig(0.0))) for p, lim in zip(prompts, limits)]
    eng.run_until_idle()
    cached = [eng.result(j).cached_tokens for j in ids]
    # nothing yet; 3 pages; at least the last token is fed (7 usable tokens: 1 page) and so is the row the limit of 9 leaves;
    # 2 pages of the 8 usable tokens; another first token: no prefix
    assert cached == [0, 12, 4, 8, 0]
    for j, p, lim in zip(ids, prompts, limits):
        assert eng.result(j).generated_tokens == alone(p, lim, SamplerConfig(0.0), ())[0]
    for j, p in zip(ids, prompts):                                                 # what was cached was not fed again
        rows = sum(n for e in runner.log for r, n, _ in e if r == ("job", j))
        new_prompt_rows = min(len(p), eng.jobs[j].steps) - eng.result(j).cached_tokens
        assert new_prompt_rows <= rows <= new_prompt_rows + len(eng.result(j).generated_tokens)
    assert eng.stats.prefix_hits == 3 and eng.stats.prefix_tokens == 24
    assert pages_when_forgotten(runner) == [32]


def test_pages_only_the_prefix_index_holds_are_given_back_before_anyone_is_preempted():
    runner = FakeRunner(page_size=4, n_pages=8, max_rows=64)                       # 32 positions
    eng = Engine(runner, EngineConfig(max_running=2), sample=host_sample)
    a = eng.submit(EngineRequest(list(range(1, 17)), 20, SamplerConfig(0.0)))      # fills 5 pages, 4 of them stay named
    eng.run_until_idle()
    assert len(eng.prefix) == 5 and runner.cache.free_pages() == [3]
    b = eng.submit(EngineRequest(list(range(30, 48)), 30, SamplerConfig(0.0)))     # needs 8 pages in the end
    eng.run_until_idle()
    assert eng.result(b).error == "" and eng.stats.preemptions == 0 and eng.stats.evicted_pages == 5
    assert eng.result(b).generated_tokens == alone(list(range(30, 48)), 30, SamplerConfig(0.0), ())[0]
    assert pages_when_forgotten(runner) == [8]


def test_prefix_sharing_can_be_switched_off_and_is_off_where_the_cache_cannot_share():
    eng = Engine(FakeRunner(), EngineConfig(prefix_cache=False), sample=host_sample)
    assert eng.prefix is None
    j = eng.submit(EngineRequest([1] * 9, 12, SamplerConfig(0.0)))
    k = eng.submit(EngineRequest([1] * 9, 12, SamplerConfig(0.0)))
    eng.run_until_idle()
    assert eng.result(k).cached_tokens == 0 and eng.result(j).generated_tokens == eng.result(k).generated_tokens
    assert Engine(FakeRunner(windows=True), sample=host_sample).prefix is None     # a windowed group gives pages back early


def test_step_uploads_ring_on_the_cpu():
    """The ring that carries a step's int32 data: pieces are snapshots, start at 16-byte multiples, keep their
    values while later steps fill other buffers, and what exceeds the ring is copied the ordinary way."""
    import numpy as np
    from geneinfer_amd.engine.runner import _StepUploads
    ring = _StepUploads("cpu", capacity=32)
    kept = []
    for step in range(2 * _StepUploads.DEPTH):
        ring.begin_step()
        a = np.arange(5, dtype=np.int32) + 100 * step
        piece = ring.put(a)
        a[:] = -1                                             # the caller may reuse its array at once
        second = ring.put(np.full((2, 3), step, dtype=np.int64))
        staged = ring.stage([step, step + 1])
        assert piece.tolist() == [100 * step + i for i in range(5)] and second.tolist() == [step] * 6 and staged.tolist() == [step, step + 1]
        assert piece.dtype == second.dtype == staged.dtype == torch.int32
        assert ring.used % 4 == 0 and piece.data_ptr() % 16 == second.data_ptr() % 16
        big = ring.put(np.arange(100, dtype=np.int32))        # more than the ring holds
        assert big.tolist() == list(range(100))
        x, y = ring.put(np.arange(3), np.arange(7) + step)    # several at once: one copy, each piece aligned
        assert x.tolist() == [0, 1, 2] and y.tolist() == [step + i for i in range(7)] and y.data_ptr() % 16 == x.data_ptr() % 16
        used = ring.used
        x, y = ring.put(np.arange(3), np.arange(100))         # ... and when one of them does not fit, nothing of the ring is used
        assert x.tolist() == [0, 1, 2] and y.tolist() == list(range(100)) and ring.used == used
        ring.end_step()
        kept.append((step, piece))
        for s, p in kept[-(_StepUploads.DEPTH - 1):]:         # the pieces of the last steps are still what they were
            assert p.tolist() == [100 * s + i for i in range(5)]


def test_pages_the_prefix_index_keeps_serve_whoever_reserves_next():
    """The index belongs to the cache manager and outlives the scheduler that filled it: on a pool that only fits after
    index-only pages are taken back, a lone `generate`, a scheduler without prefix sharing and a bare reservation all
    run, and none of them finds the pool too small."""
    runner = FakeRunner(page_size=4, n_pages=8, max_requests=2, max_positions=32)
    filler = Engine(runner, EngineConfig(max_running=1, prefix_cache=True), sample=host_sample)
    prompt = list(range(1, 27))
    filler.submit(EngineRequest(prompt, 28, SamplerConfig(temperature=0.0)))
    filler.run_until_idle()
    cache = runner.cache
    assert cache.prefix is not None and cache.evictable_pages() == 7 and cache.free_pages() == [1]      # 28 positions: 7 full pages stay named
    # a lone request through the single-request loop
    other = [40 + i % 9 for i in range(20)]
    got = generate(runner, Sampler(SamplerConfig(temperature=0.0), VOCAB), other, 24, sample=host_sample_row)
    assert got.generated_tokens == alone(other, 24, SamplerConfig(temperature=0.0), ())[0]
    assert cache.evicted_pages >= 5
    # refill the index, then a scheduler that does not share prefixes
    filler.submit(EngineRequest(prompt, 28, SamplerConfig(temperature=0.0)))
    filler.run_until_idle()
    assert cache.free_pages()[0] + cache.evictable_pages() == 8 and cache.evictable_pages() >= 6
    plain = Engine(runner, EngineConfig(max_running=1, prefix_cache=False), sample=host_sample)
    jid = plain.submit(EngineRequest(other, 24, SamplerConfig(temperature=0.0)))
    plain.run_until_idle()
    assert plain.result(jid).error == "" and plain.result(jid).generated_tokens == got.generated_tokens
    assert plain.stats.evicted_pages > 0
    # and a bare reservation
    filler.submit(EngineRequest(prompt, 28, SamplerConfig(temperature=0.0)))
    filler.run_until_idle()
    runner.open("bare")
    runner.open("second")
    assert cache.fits([("bare", 26)]) and not cache.fits([("bare", 26), ("second", 5)])
    cache.reserve([("bare", 26)])
    cache.advance("bare", 26)
    cache.check_consistency()
    with pytest.raises(OutOfPages):
        cache.reserve([("second", 5)])
    cache.reserve([("second", 4)])
    runner.close("bare")
    runner.close("second")
    assert pages_when_forgotten(runner) == [8]
