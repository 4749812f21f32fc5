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

    def open(self, r):
        self.cache.open(r)
        self.fed[r] = []

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
                self.fed[e.request].append(int(t))
                if i in e.want:
                    seed = int.from_bytes(hashlib.sha256(str(self.fed[e.request]).encode()).digest()[:8], "little")
                    rows.append(np.random.default_rng(seed).standard_normal(VOCAB).astype(np.float32) * 2)
            self.cache.advance(e.request, len(e.tokens))
        self.log.append([(e.request, len(e.tokens), tuple(e.want)) for e in entries])
        self.cache.check_consistency()
        return torch.from_numpy(np.stack(rows)) if rows else None


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
def test_every_request_gets_the_tokens_it_gets_alone(n_pages, max_running, step_rows, chunk):      # src/runtime/engine.h:8-9, tools/engine_check_main.cpp:179-211
    rng = random.Random(n_pages * 100 + max_running)
    requests = make_requests(rng, 9)
    runner = FakeRunner(n_pages=n_pages, max_requests=8, max_rows=64)
    eng = Engine(runner, EngineConfig(max_running, step_rows, chunk), END, sample=host_sample)
    ids = [eng.submit(EngineRequest(p, limit, cfg)) for p, limit, cfg in requests[:5]]
    for _ in range(3):                                                 # the rest arrive while the first are running
        eng.step()
    ids += [eng.submit(EngineRequest(p, limit, cfg)) for p, limit, cfg in requests[5:]]
    eng.run_until_idle()
    assert eng.idle() and not runner.cache.open_requests()
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
    print(f"pages {n_pages}: {st.passes} passes, {st.preemptions} preemptions")
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
    assert runner.cache.free_pages() == [6]


def test_a_lone_request_that_cannot_fit_fails_with_the_reference_message():        # src/runtime/engine.cpp:157-163
    runner = FakeRunner(page_size=4, n_pages=3, max_rows=64)
    eng = Engine(runner, sample=host_sample)
    big = eng.submit(EngineRequest([3] * 8, 40, SamplerConfig(0.0)))
    eng.run_until_idle()
    r = eng.result(big)
    assert r.finished and r.error == POOL_TOO_SMALL and len(r.generated_tokens) == 12 - 8 + 1
    assert runner.cache.free_pages() == [3]
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
        ring.end_step()
        kept.append((step, piece))
        for s, p in kept[-(_StepUploads.DEPTH - 1):]:         # the pieces of the last steps are still what they were
            assert p.tolist() == [100 * s + i for i in range(5)]
