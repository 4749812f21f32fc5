"""The scheduler: continuous batching above the step function.

Policy, as the reference's engine (src/runtime/engine.cpp:64-205):
  * admission: first come first served while fewer than `max_running` requests run; admission
    does not look at free memory.
  * a step has a budget of `step_rows` rows.  First every request with exactly one pending token
    (decoding, or at the last token of its prompt) gets one row, in admission order; then the
    others get a portion of their prompt, oldest first, of at most `prefill_chunk` rows.  A
    portion is shortened until its new pages fit in the free pages.
  * when no row fits: a lone request is finished with the error "the KV pool is too small for
    this request"; otherwise the youngest running request is preempted: its pages are freed,
    it goes to the front of the waiting queue and is later fed again from its first token,
    prompt and generated tokens alike, with its sampler's state kept, so that it continues as if
    nothing had happened.
  * prefix sharing (on unless the configuration or the model's cache rules it out): a request that starts with
    tokens an earlier request has processed takes that request's full pages and is fed from there (at least its
    last token is always fed: it produces the logits).  The index of such pages belongs to the cache manager and
    outlives the scheduler that filled it; pages only the index still holds count as free when rows are planned,
    and any reservation that needs them takes them back (this scheduler's, another one's on the same runner, a lone
    `generate`).  A preempted request is closed like any other, so what it had computed usually serves it again
    when it returns.
  * with `portion_quantum` > 0 a portion that the budget (not the prompt's end) cuts short is cut at a multiple of that many rows
    (ours, not the reference's: steps of one shape can be replayed from a captured pass, see `Runner`).
  * only the row of a request's last known token returns logits; the request's own sampler draws
    the next token from them.  A sampled end token finishes the request (it stays the last
    generated token); so does reaching `max_positions` (prompt plus generated tokens).
  * decoding ahead (on where the runner can take a step's tokens from the device): while every running request
    decodes and no other can be admitted, the next step is put in the queue before the host has read the tokens of the
    last one (they go from the sampling kernel straight into the next step), so the device does not wait for the
    host between steps.  A request that turns out to have ended (an end token) has one row too many computed, which
    nobody sees; ends by length are known beforehand.  Admission, portions of prompts, filtered sampling and a
    shortage of pages all fall back to steps whose tokens are read before the next one is planned.
Each request gets the tokens it would get alone through `generate()` with the same seed.
"""
from __future__ import annotations

from collections import deque
from dataclasses import dataclass, field
from typing import Callable, Deque, Iterable, List, Optional, Sequence

from ..cache.pages import OutOfPages
from ..sampling import Sampler, SamplerConfig, sample_rows, sample_rows_on_device
from .runner import Runner, StepEntry

POOL_TOO_SMALL = "the KV pool is too small for this request"


@dataclass
class EngineConfig:
    max_running: int = 8        # requests that hold cache memory and take part in steps at the same time
    step_rows: int = 0          # rows per step; 0 = the runner's max_rows
    prefill_chunk: int = 0      # most prompt tokens one request adds to a step; 0 = no limit besides step_rows
    prefix_cache: bool = True   # requests with equal first tokens share the pages of that prefix
    decode_ahead: bool = True   # queue the next decode step before the host has read the last one's tokens
    portion_quantum: int = 0    # > 0: a prompt portion that the budget cuts short is cut at a multiple of this many rows, so that the
                                # steps of a long prompt beside a steady batch have one shape, which the runner captures and replays
                                # (off by default: with the device as the bound it costs a few rows of every step and brings nothing)


@dataclass
class EngineRequest:
    prompt: Sequence[int]
    max_positions: int = 0                                   # prompt + generated tokens at most; 0 or too large = the context length
    sampler: SamplerConfig = field(default_factory=SamplerConfig)
    on_token: Optional[Callable[[int], None]] = None         # every generated token that is not an end token


@dataclass
class EngineResult:
    id: int = -1
    prompt_tokens: List[int] = field(default_factory=list)
    generated_tokens: List[int] = field(default_factory=list)
    finished: bool = False
    stopped_by_end_token: bool = False
    error: str = ""
    preemptions: int = 0
    cached_tokens: int = 0      # positions taken from shared pages instead of being computed (all admissions)
    first_pass: int = -1
    first_token_pass: int = -1
    last_pass: int = -1


@dataclass
class EngineStats:
    passes: int = 0
    rows: int = 0
    logits_rows: int = 0
    preemptions: int = 0
    max_rows_in_pass: int = 0
    max_chunk: int = 0
    max_running_seen: int = 0
    prefix_tokens: int = 0      # positions served by shared pages
    prefix_hits: int = 0        # admissions that found at least one shared page
    evicted_pages: int = 0


class _Job:
    def __init__(self, jid: int, request: EngineRequest, sampler: Sampler, steps: int):
        self.id, self.request, self.sampler, self.steps = jid, request, sampler, steps
        self.tokens: List[int] = [int(t) for t in request.prompt]      # prompt followed by generated tokens
        self.fed = 0                                                     # tokens[0:fed] are in the cache
        self.indexed_upto = 0                                            # ... and tokens[0:indexed_upto] known to the prefix index,
        self.indexed_after = None                                        # ... whose walk ended here (`PrefixIndex.last_walk`)
        self.result = EngineResult(id=jid, prompt_tokens=list(self.tokens))
        self.key = ("job", jid)


class _Flight:
    """A decode step in the queue whose tokens the host has not read yet."""

    def __init__(self, taken, tokens, host, ready, pass_no):
        self.taken, self.tokens, self.host, self.ready, self.pass_no = taken, tokens, host, ready, pass_no      # taken: [(job, rows)]


class Engine:
    def __init__(self, runner: Runner, config: Optional[EngineConfig] = None, end_tokens: Iterable[int] = (), sample=sample_rows):
        """`sample(logits, samplers) -> tokens` draws one token per row of logits with that row's sampler."""
        cfg = config or EngineConfig()
        self._sample = sample
        if cfg.max_running < 1:
            raise ValueError("Engine: max_running must be >= 1")
        if cfg.step_rows < 0 or cfg.prefill_chunk < 0:
            raise ValueError("Engine: step_rows and prefill_chunk must be >= 0")
        step_rows = cfg.step_rows if 0 < cfg.step_rows <= runner.max_rows else runner.max_rows
        self.cfg = EngineConfig(min(cfg.max_running, runner.cache.max_requests), step_rows, cfg.prefill_chunk or step_rows, cfg.prefix_cache,
                                cfg.decode_ahead, max(0, cfg.portion_quantum))
        self.runner = runner
        self.prefix = runner.cache.prefix if cfg.prefix_cache and runner.cache.enable_prefix_sharing() else None
        self.end_tokens = set(int(t) for t in end_tokens)
        self.jobs: List[_Job] = []
        self.waiting: Deque[_Job] = deque()
        self.running: List[_Job] = []                                    # in admission order
        self.stats = EngineStats()
        self._evicted_before = runner.cache.evicted_pages
        # decoding ahead: the step in the queue, and two pinned buffers its tokens come back through in turn
        self._flight: Optional[_Flight] = None
        self._landing_strips, self._strip = None, 0
        if cfg.decode_ahead and sample is sample_rows and hasattr(runner, "step_from_device"):
            import torch
            if torch.device(runner.model.device).type == "cuda":
                self._landing_strips = [torch.empty(self.cfg.max_running, dtype=torch.int32, pin_memory=True) for _ in range(2)]

    # ----------------------------------------------------------------------------- interface
    def submit(self, request: EngineRequest) -> int:
        context, vocab = self.runner.max_positions, self.runner.model.spec.vocab_size
        if len(request.prompt) == 0:
            raise ValueError("Engine.submit: prompt has no tokens")
        if len(request.prompt) > context:
            raise ValueError(f"Engine.submit: prompt of {len(request.prompt)} tokens does not fit in the context length {context}")
        if any(not 0 <= int(t) < vocab for t in request.prompt):
            raise ValueError("Engine.submit: token id out of range")
        sampler = Sampler(request.sampler, vocab)                         # validates the configuration
        steps = context if request.max_positions <= 0 else min(request.max_positions, context)
        job = _Job(len(self.jobs), request, sampler, steps)
        self.jobs.append(job)
        self.waiting.append(job)
        return job.id

    def idle(self) -> bool:
        return not self.waiting and not self.running and self._flight is None

    def result(self, jid: int) -> EngineResult:
        if not 0 <= jid < len(self.jobs):
            raise IndexError("Engine.result: unknown request id")
        return self.jobs[jid].result

    def run_until_idle(self) -> None:
        while self.step():
            pass

    # ------------------------------------------------------------------------------ internals
    def _admit(self) -> None:
        while self.waiting and len(self.running) < self.cfg.max_running:
            job = self.waiting.popleft()
            shared = []
            if self.prefix is not None:
                # at least one token must still be fed (it produces the logits), and the position limit must leave a row
                usable = min(len(job.tokens) - 1, job.steps - 1)
                shared = self.prefix.match(job.tokens, usable) if usable > 0 else []
            self.runner.open(job.key, shared)
            job.fed = job.indexed_upto = len(shared) * self.runner.cache.page_size
            job.indexed_after = None
            if shared:
                job.result.cached_tokens += job.fed
                self.stats.prefix_tokens += job.fed
                self.stats.prefix_hits += 1
            self.running.append(job)
        self.stats.max_running_seen = max(self.stats.max_running_seen, len(self.running))

    def _finish(self, job: _Job, error: str = "", pass_no: Optional[int] = None) -> None:
        job.result.finished, job.result.error, job.result.last_pass = True, error, self.stats.passes if pass_no is None else pass_no
        self.runner.close(job.key)
        self.running.remove(job)

    def _preempt_youngest(self) -> None:
        job = self.running.pop()
        self.runner.close(job.key)
        job.fed = 0
        job.result.preemptions += 1
        self.stats.preemptions += 1
        self.waiting.appendleft(job)

    def plan(self):
        """The rows of the next step: [(job, n_rows)] in step order, decoding requests first.
        Empty if not even one row fits in the free pages."""
        cache = self.runner.cache
        free = cache.available_pages()             # pages only the prefix index holds are taken back by the step's reservation
        budget = self.cfg.step_rows
        taken = []
        for phase in (0, 1):
            for job in self.running:
                pending = len(job.tokens) - job.fed
                if (phase == 0) != (pending == 1):
                    continue
                take = min(pending, job.steps - job.fed, budget, 1 if phase == 0 else self.cfg.prefill_chunk)
                if phase == 1 and self.cfg.portion_quantum and self.cfg.portion_quantum < take < pending:
                    take -= take % self.cfg.portion_quantum        # (cut by the budget, not by the prompt's end: cut at a round number)
                while take > 0 and any(n > f for n, f in zip(cache.pages_needed(job.key, take), free)):
                    take -= 1
                if take <= 0:
                    continue
                free = [f - n for f, n in zip(free, cache.pages_needed(job.key, take))]
                budget -= take
                taken.append((job, take))
        return taken

    def step(self) -> bool:
        """Runs one step.  False (and nothing done) if no request waits or runs."""
        if self._flight is not None:
            return self._step_behind_a_flight()
        self._admit()
        if not self.running:
            return False
        while True:
            taken = self.plan()
            if taken:
                break
            if len(self.running) == 1:
                self._finish(self.running[0], POOL_TOO_SMALL)
                return True
            self._preempt_youngest()

        entries, wanting = [], []
        for job, n in taken:
            last = job.fed + n == len(job.tokens)
            entries.append(StepEntry(job.key, job.tokens[job.fed:job.fed + n], (n - 1,) if last else ()))
            if last:
                wanting.append(job)
        logits = self.runner.step(entries)
        self._count_pass(taken)

        if self._landing_strips is not None and len(wanting) == len(taken) == len(self.running) and self.runner.can_step_from_device:
            # every running request decodes: its token may stay on the device for the next step
            self._flight = self._take_off(taken, sample_rows_on_device(logits, [j.sampler for j in wanting]))
            return True
        sampled = self._sample(logits, [j.sampler for j in wanting]) if wanting else []
        next_token = {j.id: t for j, t in zip(wanting, sampled)}
        for job in [job for job, n in taken if self._after_rows(job, n, next_token.get(job.id), self.stats.passes)]:
            self._finish(job)
        return True

    def _count_pass(self, taken) -> None:
        st = self.stats
        st.passes += 1
        st.evicted_pages = self.runner.cache.evicted_pages - self._evicted_before
        n_rows = sum(n for _, n in taken)
        st.rows += n_rows
        st.max_rows_in_pass = max(st.max_rows_in_pass, n_rows)
        st.max_chunk = max(st.max_chunk, max(n for _, n in taken))

    def _after_rows(self, job: _Job, n: int, nxt: Optional[int], pass_no: int) -> bool:
        """The job's books after `n` of its rows have run (and `nxt` was drawn from the last one's logits, if it
        was the job's last known token).  True if the job is finished."""
        st = self.stats
        if job.result.first_pass < 0:
            job.result.first_pass = pass_no
        job.fed += n
        if self.prefix is not None and job.fed // self.prefix.page_size > job.indexed_upto // self.prefix.page_size:
            # the pages that became full; the walk goes on where this job's last one ended, not from the first page
            self.runner.cache.index_prefix(job.key, job.tokens, job.fed, after=job.indexed_after)
            job.indexed_upto, job.indexed_after = job.fed, self.prefix.last_walk
        if nxt is not None:
            st.logits_rows += 1
            job.result.generated_tokens.append(nxt)
            job.tokens.append(nxt)
            if job.result.first_token_pass < 0:
                job.result.first_token_pass = pass_no
            if nxt in self.end_tokens:
                job.result.stopped_by_end_token = True
                return True
            if job.request.on_token is not None:
                job.request.on_token(nxt)
        return job.fed >= job.steps

    # ------------------------------------------------------------------------------ decoding ahead
    def _take_off(self, taken, tokens) -> _Flight:
        """The step's tokens (one per job of `taken`, in its order) start their way to the host, and nobody waits
        here; the step counts as in flight."""
        import torch
        host = self._landing_strips[self._strip][:len(taken)]
        self._strip ^= 1
        host.copy_(tokens, non_blocking=True)
        ready = torch.cuda.Event()
        ready.record()
        return _Flight(list(taken), tokens, host, ready, self.stats.passes)

    def _step_behind_a_flight(self) -> bool:
        """With a decode step in flight: the next one is queued with that step's tokens where they are, if the same
        requests go on for certain; then the flight's tokens are read and the requests' books brought up to date."""
        flight, ahead = self._flight, None
        jobs = [job for job, _ in flight.taken]
        goes_on = (len(jobs) == len(self.running) and not any(j.result.finished for j in jobs)          # nobody of it ended last time,
                   and all(j.fed + n < j.steps for j, n in flight.taken)                                # nobody ends by length now,
                   and (not self.waiting or len(self.running) >= self.cfg.max_running)                  # and nobody else could join
                   and self.runner.can_step_from_device)
        if goes_on:
            try:
                logits = self.runner.step_from_device([j.key for j in jobs], flight.tokens)
            except OutOfPages:                       # nothing has changed: the step after the landing sorts it out
                logits = None
            if logits is not None:
                self._count_pass([(j, 1) for j in jobs])
                ahead = self._take_off([(j, 1) for j in jobs], sample_rows_on_device(logits, [j.sampler for j in jobs]))
        flight.ready.synchronize()
        sampled = flight.host.tolist()
        finished = [job for (job, n), nxt in zip(flight.taken, sampled)
                    if not job.result.finished and self._after_rows(job, n, nxt, flight.pass_no)]
        for job in finished:                         # (a finished request's row in the step ahead is nobody's)
            self._finish(job, pass_no=flight.pass_no)
        self._flight = ahead
        return True
