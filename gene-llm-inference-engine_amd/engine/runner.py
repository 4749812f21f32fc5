"""The step function: one batch of (request, its next tokens) through the model, from the cache.

A step holds, for each of its requests, the request's next tokens: a portion of a prompt, cut
anywhere, or a single decoded token.  All rows run as one batch; positions are never passed in,
a step always appends to what the cache holds of the request.  Logits come back only for the
rows asked for.  Everything is checked before anything changes, and a step that cannot get its
pages raises `OutOfPages` and leaves every request as it was (the reference's `forward_rows`
keeps the same promises, src/model/model.h:63-76, src/model/transformer.cpp:483-518).
"""
from __future__ import annotations

import array
import gc

from dataclasses import dataclass, field
from typing import Hashable, List, Optional, Sequence

import numpy as np
import torch

from ..cache import CacheError, CacheManager
from ..kernels import ops
from ..parts import LayerCache, StepContext
from .model import DecoderModel


class StepError(ValueError):
    """The batch is not valid; nothing was changed."""


@dataclass
class StepEntry:
    request: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = field(default_factory=tuple)      # places among `tokens` whose logits are asked for
    at: Optional[int] = None                                # where the caller believes its first token goes; None: wherever the cache says


class _CacheView:
    def __init__(self, manager: CacheManager, needs, reads_from):
        self._layer = []
        for i, (need, src) in enumerate(zip(needs, reads_from)):
            from ..cache import PagedKvNeed, StateNeed
            if isinstance(need, PagedKvNeed):
                kv, table, _ = manager.kv(i)
                self._layer.append(LayerCache(kv=kv, table=table, writes=src is None))
            elif isinstance(need, StateNeed):
                self._layer.append(LayerCache(state=manager.state(i)))
            else:
                self._layer.append(LayerCache())

    def layer_cache(self, entry: int) -> LayerCache:
        return self._layer[entry]


class Runner:
    """Model + cache + the step function.

    page_size    positions per page
    max_tokens   positions the page pool holds (per layer group)
    max_requests live requests (request slots)
    max_rows     most rows one step may hold
    max_positions longest request; defaults to the model's limit
    use_graphs   replay decode steps (one token per request, all logits wanted) from captured HIP graphs,
                 if every part of the model allows it (`graph_safe`)
    graph_rows   steps of other shapes (portions of prompts, alone or beside decoded tokens) of up to this many rows are
                 captured too when their shape comes again: the same numbers of rows per request in the same order, as many
                 logits wanted, the same power-of-two bracket of the longest context (at most `max_step_graphs` are kept).
                 Such a step costs the host one copy and one launch instead of some hundred launches; longer steps keep
                 the device busy for longer than the host needs to launch them.  0: none.
    max_graphs   most captured graphs kept (one per batch size and bracket of the longest context, at least two); the
                 one used longest ago goes when another is needed.  All graphs take their memory from one pool, so what
                 they hold is what the largest of them needs (a pass's activations and its logits), not the sum.

    The logits a step returns are the caller's until the next step of this runner, of whatever batch size: captured
    steps write theirs into the graphs' common pool, where the next step's activations may lie.
    """

    def __init__(self, model: DecoderModel, *, page_size: int = 16, max_tokens: int = 4096, max_requests: int = 8,
                 max_rows: int = 4096, max_positions: Optional[int] = None, use_graphs: bool = True, max_graphs: int = 48,
                 graph_rows: int = 1024, max_step_graphs: int = 32):
        self.model = model
        self.page_size = int(page_size)
        self.max_rows = int(max_rows)
        self.max_positions = int(max_positions or model.spec.max_positions)
        needs, reads_from = model.cache_needs()
        n_pages = max(1, -(-int(max_tokens) // self.page_size))
        self.cache = CacheManager(needs, reads_from, page_size=self.page_size, n_pages=n_pages, max_requests=max_requests,
                                  max_positions=self.max_positions, dtype=model.dtype, device=model.device)
        self._view = _CacheView(self.cache, needs, reads_from)
        self.steps_run = 0
        self.rows_run = 0
        self.steps_replayed = 0                   # of them, served by the replay of a captured pass
        self.use_graphs = bool(use_graphs) and model.graph_safe
        self._graphs = {}
        self.max_graphs = max(2, int(max_graphs))       # (two at least: the graph that goes is then never the one replayed last, whose logits a step queued ahead may still be read from)
        self._graph_pool = None
        self.graph_rows = int(graph_rows)
        self.max_step_graphs = max(2, int(max_step_graphs))
        self._step_graphs = {}
        self._uploads = _StepUploads(model.device, min(8 * self.max_rows + 1024, 1 << 18))       # at most 1 MiB a buffer; what is larger is copied the ordinary way

    # -------------------------------------------------------------------------------- requests
    def open(self, request: Hashable, shared_pages: Sequence[int] = ()) -> None:
        """shared_pages: full pages of an equal prompt prefix (`CacheManager.open`)."""
        self.cache.open(request, shared_pages)

    def close(self, request: Hashable) -> None:
        self.cache.close(request)

    def truncate(self, request: Hashable, length: int) -> None:
        """Rewind: the request's next token goes to position `length` (`CacheManager.truncate`)."""
        self.cache.truncate(request, length)

    def is_open(self, request: Hashable) -> bool:
        return self.cache.is_open(request)

    def length(self, request: Hashable) -> int:
        return self.cache.length(request)

    # ------------------------------------------------------------------------------------ step
    def _validate(self, entries: Sequence[StepEntry]):
        if not entries:
            raise StepError("a step needs at least one entry")
        seen, n_rows, vocab, token_arrays = set(), 0, self.model.spec.vocab_size, []
        for e in entries:
            if e.request in seen:
                raise StepError(f"request {e.request!r} appears twice in one step")
            seen.add(e.request)
            if not self.cache.is_open(e.request):
                raise StepError(f"request {e.request!r} is not open")
            if len(e.tokens) == 0:
                raise StepError(f"request {e.request!r} brings no tokens")
            try:                                                            # (checked as a whole: a prompt portion has thousands)
                if type(e.tokens) is list:                                  # (the quickest way from a list of Python numbers to an array)
                    tokens = np.frombuffer(array.array("q", e.tokens), dtype=np.int64)
                else:
                    tokens = np.asarray(e.tokens, dtype=np.int64)
            except (TypeError, ValueError, OverflowError):
                raise StepError(f"the tokens of request {e.request!r} are not integers") from None
            if tokens.ndim != 1 or int(tokens.min()) < 0 or int(tokens.max()) >= vocab:
                bad = next((t for t in e.tokens if not 0 <= int(t) < vocab), None) if tokens.ndim == 1 else None
                raise StepError(f"token {bad} of request {e.request!r} is outside the vocabulary [0, {vocab})")
            token_arrays.append(tokens)
            for w in e.want:
                if not 0 <= int(w) < len(e.tokens):
                    raise StepError(f"request {e.request!r} wants logits at place {w} of {len(e.tokens)} tokens")
            held = self.cache.length(e.request)
            if e.at is not None and int(e.at) != held:
                # The positions are the cache's own.  A caller that names one is checked against it, in the order of
                # the reference's forward_rows (src/model/transformer.cpp:298-307): the range first, then the gap.  An earlier position is no silent rewind here: `truncate` is a call of its own.
                if int(e.at) < 0 or int(e.at) + len(e.tokens) > self.max_positions:
                    raise StepError(f"positions {int(e.at)} .. {int(e.at) + len(e.tokens) - 1} of request {e.request!r} exceed the context length {self.max_positions}")
                if int(e.at) > held:
                    raise StepError(f"a portion of request {e.request!r} at position {int(e.at)} leaves a gap: the cache holds {held} positions")
                raise StepError(f"a portion of request {e.request!r} at position {int(e.at)} lies under the {held} positions the cache holds; rewind first")
            if held + len(e.tokens) > self.max_positions:
                raise StepError(f"request {e.request!r} would pass the position limit {self.max_positions}")
            n_rows += len(e.tokens)
        if n_rows > self.max_rows:
            raise StepError(f"the step holds {n_rows} rows, more than max_rows = {self.max_rows}")
        return n_rows, token_arrays

    def step(self, entries: Sequence[StepEntry]) -> Optional[torch.Tensor]:
        """Runs the batch; returns float32 logits [wanted, vocab] on the device in the order of the
        entries and of each entry's `want`, or None if nothing was wanted.  The tensor is valid
        until the next step."""
        if self.can_step_from_device and all(len(e.tokens) == 1 and tuple(e.want) == (0,) and e.at is None for e in entries) and entries:
            return self._step_of_single_tokens(entries)
        n_rows, token_arrays = self._validate(entries)
        self.cache.reserve([(e.request, len(e.tokens)) for e in entries])       # OutOfPages: nothing changed
        self._uploads.begin_step()

        meta = np.empty((3, n_rows), dtype=np.int32)                            # tokens, positions, slots
        seg_slot, seg_start, seg_len, seg_pos0, logit_rows = [], [], [], [], []
        row = 0
        for e, tokens in zip(entries, token_arrays):
            n, slot, pos0 = len(e.tokens), self.cache.slot(e.request), self.cache.length(e.request)
            meta[0, row:row + n] = tokens
            meta[1, row:row + n] = np.arange(pos0, pos0 + n, dtype=np.int32)
            meta[2, row:row + n] = slot
            seg_slot.append(slot); seg_start.append(row); seg_len.append(n); seg_pos0.append(pos0)
            logit_rows += [row + int(w) for w in e.want]
            row += n

        dev = self.model.device
        every_row_wanted = len(logit_rows) == n_rows and logit_rows == list(range(n_rows))
        graph = self._step_graph_for(seg_len, seg_pos0, len(logit_rows), every_row_wanted)
        if graph is not None and graph.calls >= 1:           # a shape that has come before: captured now, replayed from then on
            self.cache.sync(self._uploads.put, self._uploads.stage)
            logits = graph.run(self._uploads, meta, logit_rows, seg_start, seg_len, seg_pos0, seg_slot)
            self.steps_replayed += 1
        else:
            if graph is not None:
                graph.calls += 1
            # the step's numbers and the page tables' changed columns go over in one copy: the first is only laid down, the second sends both
            if logit_rows:
                meta_dev, rows_dev = self._uploads.put(meta, np.asarray(logit_rows, dtype=np.int32), send=False)
            else:
                meta_dev, rows_dev = self._uploads.put(meta, send=False), None
            self.cache.sync(self._uploads.put, self._uploads.stage)
            self._uploads.flush()
            meta_dev = meta_dev.view(3, n_rows)
            ctx = StepContext(n_rows=n_rows, dtype=self.model.dtype, device=dev, tokens=meta_dev[0], row_pos=meta_dev[1],
                              row_slot=meta_dev[2], seg_slot=seg_slot, seg_start=seg_start, seg_len=seg_len, seg_pos0=seg_pos0,
                              upload=self._uploads.put, every_row_wanted=every_row_wanted)
            logits = self._forward(ctx, rows_dev, len(logit_rows))
        self._uploads.end_step()
        for e in entries:
            self.cache.advance(e.request, len(e.tokens))
        self.steps_run += 1
        self.rows_run += n_rows
        return logits

    def _forward(self, ctx: StepContext, rows_dev, n_logit_rows: int):
        return _pass_keeping_state(self.model, self.cache.states, ctx, self._view, rows_dev, n_logit_rows)

    # ------------------------------------------------------------------ captured steps of other shapes
    def _step_graph_for(self, seg_len, seg_pos0, n_logit_rows: int, every_row_wanted: bool):
        """The captured pass that serves a step of this shape (made at the shape's first coming, captured at its second), or
        None where such steps are not captured."""
        n_rows = sum(seg_len)
        if not (self.can_step_from_device and 0 < n_rows <= self.graph_rows):
            return None
        bracket = _context_bracket(max(p + n for p, n in zip(seg_pos0, seg_len)), self.max_positions)
        key = (tuple(seg_len), n_logit_rows, every_row_wanted, bracket)
        g = self._step_graphs.get(key)
        if g is None:
            if len(self._step_graphs) >= self.max_step_graphs:       # (never during a capture: a graph may not be freed inside one)
                del self._step_graphs[min(self._step_graphs, key=lambda k: self._step_graphs[k].last_used)]
            if self._graph_pool is None:
                self._graph_pool = torch.cuda.graph_pool_handle()
            g = self._step_graphs[key] = _StepGraph(self.model, self._view, n_rows, n_logit_rows, every_row_wanted, bracket, self._graph_pool)
        g.last_used = self.steps_run
        return g

    # --------------------------------------------------------------------------- captured decode
    @property
    def can_step_from_device(self) -> bool:
        """Whether `step_from_device` is served: by the captured decode step, which nobody may be watching from the
        inside (a trace of the layers, a timing of the kernels)."""
        return bool(self.use_graphs) and self.model.trace is None and not ops.profiling()

    def step_from_device(self, requests: Sequence[Hashable], tokens: torch.Tensor) -> torch.Tensor:
        """A decode step whose tokens are still on the device: request i brings `tokens[i]` (int32, typically what the
        sampler made of the previous step's logits and nobody has waited for yet) and wants its logits.  The caller
        can so put the next step in the queue before the host knows the last one's tokens.  The tokens are not
        checked against the vocabulary (a sampler makes none outside it); everything else is `step`'s."""
        if not self.can_step_from_device:
            raise StepError("tokens on the device are taken by the captured decode step only")
        if not (tokens.dtype == torch.int32 and tokens.shape == (len(requests),) and tokens.device == torch.device(self.model.device)):
            raise StepError("step_from_device: tokens must be int32 [requests] on the model's device")
        return self._step_of_single_tokens([StepEntry(r, [0], (0,)) for r in requests], tokens)

    def _step_of_single_tokens(self, entries: Sequence[StepEntry], tokens_on_device: Optional[torch.Tensor] = None) -> torch.Tensor:
        """The decode step: every request brings one token and wants its logits.  The same checks and the
        same bookkeeping as the general path, done over whole lists at once (this path runs once per
        generated token of every request, so its host time counts)."""
        cache, n = self.cache, len(entries)
        requests = [e.request for e in entries]
        if len(set(requests)) != n:
            raise StepError("a request appears twice in one step")
        try:
            slots, lengths = cache.slots_and_lengths(requests)
        except CacheError as err:
            raise StepError(str(err)) from None
        tokens = [int(e.tokens[0]) for e in entries]
        vocab = self.model.spec.vocab_size
        if min(tokens) < 0 or max(tokens) >= vocab:
            bad = next(i for i, t in enumerate(tokens) if not 0 <= t < vocab)
            raise StepError(f"token {tokens[bad]} of request {requests[bad]!r} is outside the vocabulary [0, {vocab})")
        if max(lengths) + 1 > self.max_positions:
            bad = max(range(n), key=lengths.__getitem__)
            raise StepError(f"request {requests[bad]!r} would pass the position limit {self.max_positions}")
        if n > self.max_rows:
            raise StepError(f"the step holds {n} rows, more than max_rows = {self.max_rows}")
        cache.reserve_one_each(requests, slots, lengths)                        # OutOfPages: nothing changed
        self._uploads.begin_step()
        cache.sync(self._uploads.put, self._uploads.stage)
        # Captured steps exist for some batch sizes only: rows of the spare slot, at position 0, fill the step up to the next of them.
        fill = captured_batch_size(n, self.max_rows) - n
        if fill:
            tokens, lengths, slots = tokens + [0] * fill, lengths + [0] * fill, slots + [cache.spare_slot] * fill
        meta = self._uploads.stage(np.array([tokens, lengths, slots], dtype=np.int32)).view(3, n + fill)
        logits = self._decode_step(meta, slots, lengths, tokens_on_device)[:n]
        self._uploads.end_step()
        cache.advance_one_each(requests, slots[:n], lengths[:n])
        self.steps_run += 1
        self.rows_run += n
        return logits

    def _decode_step(self, meta: torch.Tensor, seg_slot, seg_pos0, tokens_on_device=None) -> torch.Tensor:
        """A step in which every request brings one token and wants its logits runs as a replay of a
        HIP graph captured once per batch size: the launches of the whole pass cost one call.  The
        graph reads tokens, positions and slots from fixed device buffers that are filled before
        every replay; nothing else in it depends on the step."""
        batch = meta.shape[1]
        # The attention kernel's cut of the context into pieces is fixed at capture, for the longest context the graph
        # is to serve well: one graph per batch size and power-of-two bracket of the step's longest context.
        bracket = _context_bracket(max(seg_pos0) + 1, self.max_positions)
        g = self._graphs.get((batch, bracket))
        if g is None:
            if len(self._graphs) >= self.max_graphs:         # (never during a capture: a graph may not be freed inside one)
                del self._graphs[min(self._graphs, key=lambda k: self._graphs[k].last_used)]
            if self._graph_pool is None:
                self._graph_pool = torch.cuda.graph_pool_handle()
            g = self._graphs[(batch, bracket)] = _DecodeGraph(self.model, self._view, bracket, batch, self._graph_pool, self.cache.states)
        g.last_used = self.steps_run
        self.steps_replayed += 1 if g.calls >= 1 else 0
        return g.run(meta, seg_slot, seg_pos0, tokens_on_device)


def _pass_keeping_state(model: DecoderModel, states, ctx: StepContext, view, rows_dev, n_logit_rows: int):
    """The pass, launched kernel by kernel.  Fixed-size state is committed only by a pass that succeeds: parts write their
    state slots as they go, so the slots of the step's requests are kept aside first and put back if the pass raises (the
    requests' lengths have not moved yet, and pages reserved for the step stay with their requests for the next try).  A
    pass that is being captured changes nothing if it raises, and a replay runs no code of the parts."""
    if not states:
        return model.forward(ctx, view, rows_dev, n_logit_rows)
    slots = torch.tensor(sorted(set(ctx.seg_slot)), dtype=torch.int64, device=model.device)
    kept = {entry: state.index_select(0, slots) for entry, state in states.items()}
    try:
        return model.forward(ctx, view, rows_dev, n_logit_rows)
    except BaseException:
        for entry, state in states.items():
            state.index_copy_(0, slots, kept[entry])
        raise


def _context_bracket(longest: int, most: int) -> int:
    """The power of two from 1,024 on that holds `longest` positions (at most `most`): what a captured pass is made for."""
    bracket = 1024
    while bracket < longest:
        bracket *= 2
    return min(bracket, most)


def captured_batch_size(n: int, most: int) -> int:
    """The batch size of the captured decode step that serves n rows: every size up to 8, then multiples of 2 up to 16, of 4
    up to 64, of 8 up to 128 and of 16 beyond, so that a batch that shrinks request by request as they finish, or grows as they are
    admitted, meets a few dozen graphs instead of one per size (capturing one costs several steps' time); the added rows
    are at most a fifth of the step and cost next to nothing (one key each).  Never more than `most` rows."""
    step = 1 if n <= 8 else 2 if n <= 16 else 4 if n <= 64 else 8 if n <= 128 else 16
    size = -(-n // step) * step
    return size if size <= most else n


class _StepUploads:
    """The int32 data a step makes on the host (tokens, positions, slots, row lists, tile lists) goes to
    the device through pinned memory with copies that do not wait: a ring of buffers, one per step in
    flight; a buffer is taken again only after the copies of its last use have finished.  What `put`
    returns is valid while the step runs."""
    DEPTH = 4

    def __init__(self, device, capacity: int):
        self.device, self.capacity = device, capacity
        on_gpu = torch.device(device).type == "cuda"
        self.host = [torch.empty(capacity, dtype=torch.int32, pin_memory=on_gpu) for _ in range(self.DEPTH)]
        self.host_np = [h.numpy() for h in self.host]            # the same memory, for numpy to write into
        self.dev = [torch.empty(capacity, dtype=torch.int32, device=device) for _ in range(self.DEPTH)]
        self.done = [None] * self.DEPTH
        self.turn, self.used, self.sent = 0, 0, 0

    def begin_step(self) -> None:
        self.turn = (self.turn + 1) % self.DEPTH
        self.used, self.sent = 0, 0
        if self.done[self.turn] is not None:
            self.done[self.turn].synchronize()

    def put(self, *arrays, send: bool = True):
        """The arrays on the device (int32, flattened): one tensor for one array, a tuple for several, which then
        go over in one copy.  send=False only lays them down in the pinned buffer: they go over with the next `put`
        that sends, or with `flush`, and what is returned is valid from then on."""
        flats = [np.ascontiguousarray(values, dtype=np.int32).reshape(-1) for values in arrays]
        first, spans = self.used, []
        for flat in flats:
            a = self.used
            if a + flat.size > self.capacity:                   # more than the ring was made for: ordinary copies
                self.used = first
                pieces = tuple(torch.from_numpy(f.copy()).to(self.device) for f in flats)
                return pieces[0] if len(pieces) == 1 else pieces
            self.host_np[self.turn][a:a + flat.size] = flat
            spans.append((a, a + flat.size))
            self.used = (a + flat.size + 3) & ~3                # pieces start at multiples of 16 bytes
        if send:
            self.flush()
        pieces = tuple(self.dev[self.turn][a:b] for a, b in spans)
        return pieces[0] if len(pieces) == 1 else pieces

    def flush(self) -> None:
        """Sends what has been laid down since the last copy."""
        if self.used > self.sent:
            self.dev[self.turn][self.sent:self.used].copy_(self.host[self.turn][self.sent:self.used], non_blocking=True)
            self.sent = self.used

    def stage(self, values: np.ndarray) -> torch.Tensor:
        """The values in this step's pinned buffer only (for a copy the caller makes itself, into its own device memory)."""
        flat = np.ascontiguousarray(values, dtype=np.int32).reshape(-1)
        n = flat.size
        if self.used + n > self.capacity:
            return torch.from_numpy(flat.copy())
        a, b = self.used, self.used + n
        self.used = (b + 3) & ~3
        if self.sent == a:                                      # (not the ring's to send)
            self.sent = self.used
        self.host_np[self.turn][a:b] = flat
        return self.host[self.turn][a:b]

    def region(self, n: int) -> torch.Tensor:
        """n ints of this step's pinned buffer in one piece, for a caller that lays several arrays out itself and copies them
        over at once."""
        if self.used + n > self.capacity:
            return torch.empty(n, dtype=torch.int32, pin_memory=torch.device(self.device).type == "cuda")
        a = self.used
        self.used = (a + n + 3) & ~3
        if self.sent == a:
            self.sent = self.used
        return self.host[self.turn][a:a + n]

    def end_step(self) -> None:
        if torch.device(self.device).type == "cuda":
            ev = self.done[self.turn] or torch.cuda.Event()
            ev.record()
            self.done[self.turn] = ev


class _DecodeGraph:
    """The captured pass of one batch size.  The logits a replay returns lie in the graphs' common pool: they are the
    caller's until the next step, whichever graph that step replays.  It holds the model and the cache view, not the runner: a runner and
    its graphs must not form a reference cycle, or they would be freed by the cycle collector at a moment of its
    choosing, possibly while another graph is being captured, which the HIP runtime answers by aborting."""

    def __init__(self, model: DecoderModel, view, longest_context: int, batch: int, pool=None, states=None):
        from ..kernels.ops import AttentionPlan
        self.model, self.view, self.batch, self.pool, self.last_used, self.states = model, view, batch, pool, 0, states
        dev = model.device
        self.meta = torch.zeros((3, batch), dtype=torch.int32, device=dev)
        self.logit_rows = torch.arange(batch, dtype=torch.int32, device=dev)
        self.plan = AttentionPlan.all_decode(batch, longest_context, dev)
        self.graph = None
        self.logits = None
        self.calls = 0

    def _context(self, seg_slot, seg_pos0) -> StepContext:
        m, b = self.model, self.batch
        ctx = StepContext(n_rows=b, dtype=m.dtype, device=m.device, tokens=self.meta[0], row_pos=self.meta[1], row_slot=self.meta[2],
                          seg_slot=list(seg_slot), seg_start=list(range(b)), seg_len=[1] * b, seg_pos0=list(seg_pos0), every_row_wanted=True)
        ctx.memo["attention_plan"] = self.plan
        return ctx

    def run(self, meta: torch.Tensor, seg_slot, seg_pos0, tokens_on_device=None) -> torch.Tensor:
        """meta: this step's tokens, positions and slots, int32 [3, batch], in pinned memory that stays as it is
        until the copy made here has run.  tokens_on_device: the tokens, if the host does not know them yet."""
        self.meta.copy_(meta, non_blocking=True)
        if tokens_on_device is not None:                 # (of the requests' rows; rows that fill the step up come behind them)
            self.meta[0, :tokens_on_device.shape[0]].copy_(tokens_on_device, non_blocking=True)
        self.calls += 1
        if self.graph is None:
            if self.calls < 2:          # the first step of a batch size runs as it is; a size that comes again is captured
                return _pass_keeping_state(self.model, self.states, self._context(seg_slot, seg_pos0), self.view, self.logit_rows, self.batch)
            # Capturing records the launches without running them, so this step runs once more below, by replay.
            # No garbage collection meanwhile: freeing device memory or another graph inside a capture aborts.
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            collecting = gc.isenabled()
            gc.disable()
            try:
                with torch.cuda.graph(graph, pool=self.pool):
                    self.logits = self.model.forward(self._context(seg_slot, seg_pos0), self.view, self.logit_rows, self.batch)
            finally:
                if collecting:
                    gc.enable()
            self.graph = graph
        self.graph.replay()
        return self.logits


class _StepGraph:
    """The captured pass of one step shape other than the all-decode one: the same numbers of rows per request in the same order
    (portions of prompts, alone or beside decoded tokens), as many logits wanted, one bracket of the longest context.  Everything
    the pass reads of the step (tokens, positions, slots, the rows whose logits are wanted, the attention's lists of tiles and
    rows) lies in one block of device memory at places the shape fixes; a step lays its numbers out in pinned memory, sends them
    over in one copy and replays.  The attention cuts contexts for the bracket's longest (`AttentionPlan` with its two context
    lengths set to the bracket), as the captured decode step does."""

    def __init__(self, model: DecoderModel, view, n_rows: int, n_logit_rows: int, every_row_wanted: bool, bracket: int, pool):
        self.model, self.view, self.n_rows, self.n_logit_rows, self.every_row_wanted = model, view, n_rows, n_logit_rows, every_row_wanted
        self.bracket, self.pool = bracket, pool
        self.block, self.places = None, None                 # the device block, and where each array lies in it: [(offset, size)]
        self.graph, self.logits, self.calls, self.last_used = None, None, 0, 0

    def _lay_out(self, uploads, meta, logit_rows, seg_start, seg_len, seg_pos0, seg_slot) -> StepContext:
        """The step's numbers into the block (one copy, nobody waits), and the pass's context over the block's views."""
        from ..kernels.ops import AttentionPlan
        arrays = [np.ascontiguousarray(meta, dtype=np.int32).reshape(-1)]
        if self.n_logit_rows:
            arrays.append(np.asarray(logit_rows, dtype=np.int32))
        first_of_plan = len(arrays)

        def collect(*lists):                                 # the attention plan's lists: kept for the copy below, views handed back
            for values in lists:
                arrays.append(np.asarray(values, dtype=np.int32).reshape(-1))
            if self.places is None:
                return tuple(None for _ in lists)            # (the first time round the block does not exist yet: see below)
            return tuple(self._view(first_of_plan + i) for i in range(len(lists)))

        plan = AttentionPlan(seg_start, seg_len, seg_pos0, seg_slot, self.model.device, to_device=collect)
        if self.places is None:                              # the shape's layout, fixed from now on: every array at a multiple of 16 bytes
            offset, places = 0, []
            for a in arrays:
                places.append((offset, a.size))
                offset = (offset + a.size + 3) & ~3
            self.places, self.block = places, torch.zeros(max(offset, 4), dtype=torch.int32, device=self.model.device)
            if plan.n_tiles:
                plan.tiles, plan.tile_first, plan.tile_rows = self._view(first_of_plan), self._view(first_of_plan + 1), self._view(first_of_plan + 2)
                plan.decode_rows = self._view(first_of_plan + 3) if len(arrays) > first_of_plan + 3 else None
        if [a.size for a in arrays] != [size for _, size in self.places]:
            raise StepError("a captured step met a step of another shape")          # (the shape's key should have told them apart)
        total = self.places[-1][0] + self.places[-1][1]
        staged = uploads.region(total)
        flat = staged.numpy()
        for a, (offset, size) in zip(arrays, self.places):
            flat[offset:offset + size] = a
        self.block[:total].copy_(staged, non_blocking=True)
        if plan.n_tiles:
            plan.max_tile_context = self.bracket
        if plan.n_decode:
            plan.max_decode_context = self.bracket
        m = self.model
        meta_dev = self._view(0).view(3, self.n_rows)
        ctx = StepContext(n_rows=self.n_rows, dtype=m.dtype, device=m.device, tokens=meta_dev[0], row_pos=meta_dev[1], row_slot=meta_dev[2],
                          seg_slot=list(seg_slot), seg_start=list(seg_start), seg_len=list(seg_len), seg_pos0=list(seg_pos0),
                          every_row_wanted=self.every_row_wanted)
        ctx.memo["attention_plan"] = plan
        return ctx

    def _view(self, i: int) -> torch.Tensor:
        offset, size = self.places[i]
        return self.block[offset:offset + size]

    def run(self, uploads, meta, logit_rows, seg_start, seg_len, seg_pos0, seg_slot):
        ctx = self._lay_out(uploads, meta, logit_rows, seg_start, seg_len, seg_pos0, seg_slot)
        self.calls += 1
        if self.graph is None:
            rows_dev = self._view(1) if self.n_logit_rows else None
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            collecting = gc.isenabled()
            gc.disable()                                     # (freeing device memory or another graph inside a capture aborts)
            try:
                with torch.cuda.graph(graph, pool=self.pool):
                    self.logits = self.model.forward(ctx, self.view, rows_dev, self.n_logit_rows)
            finally:
                if collecting:
                    gc.enable()
            self.graph = graph
        self.graph.replay()
        return self.logits
