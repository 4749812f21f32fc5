"""From logits to the next token: greedy, temperature, top-k, top-p, with the reference's random
generator, so that a seed gives the same stream of uniform numbers as there.

Rules (src/sampler/sampler.h:1-14, src/sampler/sampler.cpp:25-129):
  1. temperature <= 0: the largest logit wins, the lowest index among equals; no randomness is used.
  2. otherwise p = softmax(logits / temperature).
  3. top-k keeps the k most likely tokens, top-p then the shortest prefix (by probability
     descending, index ascending) whose mass reaches top_p times the kept mass.
  4. a token is drawn by walking the kept tokens until the cumulative probability exceeds
     u times the kept mass; without filtering the walk is in index order.
All of it runs on the device, on the logits where the step left them; `filtered_draw` states
steps 2-4 on the host as the reference has them, for one row.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import List, Sequence

import numpy as np
import torch

from ..kernels import ops

_MASK = (1 << 64) - 1


@dataclass(frozen=True)
class SamplerConfig:
    temperature: float = 0.8      # <= 0 means greedy
    top_k: int = 0                # 0 = off
    top_p: float = 1.0            # 1 = off; in (0, 1]
    seed: int = 1

    def validate(self, vocab_size: int) -> None:
        if vocab_size <= 0:
            raise ValueError("sampler: vocab_size must be positive")
        if not self.temperature >= 0.0:                       # also refuses NaN
            raise ValueError("sampler: temperature must be >= 0")
        if self.top_k < 0:
            raise ValueError("sampler: top_k must be >= 0")
        if not 0.0 < self.top_p <= 1.0:
            raise ValueError("sampler: top_p must be in (0, 1]")

    @property
    def greedy(self) -> bool:
        return self.temperature <= 0.0

    def filters(self, vocab_size: int) -> bool:
        return 0 < self.top_k < vocab_size or self.top_p < 1.0


def _splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _MASK
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & _MASK
    return x ^ (x >> 31)


class UniformStream:
    """xorshift64* started from splitmix64(seed); 24 random bits give u in [0, 1)."""

    def __init__(self, seed: int):
        self.state = _splitmix64(int(seed) & _MASK) or 1

    def next_u32(self) -> int:
        s = self.state
        s ^= s >> 12
        s ^= (s << 25) & _MASK
        s ^= s >> 27
        self.state = s
        return ((s * 0x2545F4914F6CDD1D) & _MASK) >> 32

    def next_uniform(self) -> float:
        return (self.next_u32() >> 8) / 16777216.0


def filtered_draw(logits: np.ndarray, cfg: SamplerConfig, u: float) -> int:
    """Steps 2-4 on the host for one row (float32 probabilities, float64 sums)."""
    logits = np.asarray(logits, dtype=np.float32)
    n = logits.shape[0]
    p = np.exp((logits - logits.max()) / np.float32(cfg.temperature), dtype=np.float32)
    p *= np.float32(1.0 / float(p.sum(dtype=np.float64)))
    order = np.arange(n)
    if cfg.filters(n):
        order = np.lexsort((order, -p))                       # probability descending, index ascending
        if 0 < cfg.top_k < n:
            order = order[:cfg.top_k]
        if cfg.top_p < 1.0:
            cum = np.cumsum(p[order], dtype=np.float64)
            reached = np.nonzero(cum >= float(np.float32(cfg.top_p)) * cum[-1])[0]
            if reached.size:
                order = order[:reached[0] + 1]
    cum = np.cumsum(p[order], dtype=np.float64)
    hit = np.nonzero(float(np.float32(u)) * cum[-1] < cum)[0]
    return int(order[hit[0]] if hit.size else order[-1])


class Sampler:
    """One request's sampler: its configuration and its own stream of uniform numbers."""

    def __init__(self, config: SamplerConfig, vocab_size: int):
        config.validate(vocab_size)
        self.config, self.vocab_size = config, vocab_size
        self.stream = UniformStream(config.seed)
        # which kernels this sampler's rows go through in `sample_rows`: arg max, plain temperature, top-k / top-p
        self.kind = "greedy" if config.greedy else "filtered" if config.filters(vocab_size) else "plain"
        self.temperature = float(config.temperature)

    def next_uniform(self) -> float:
        return self.stream.next_uniform()

    def sample(self, logits: torch.Tensor) -> int:
        """One row of float32 logits on the device -> token id."""
        return sample_rows(logits.reshape(1, -1), [self])[0]


_KIND_ORDER = {"greedy": 0, "plain": 1, "filtered": 2}


class _Staging:
    """The rows' parameters go to the device through pinned memory with a copy that does not wait.  (A copy from ordinary
    memory makes the host wait until the device has reached it, that is until the step before it has run: the host could then
    queue nothing ahead.)  A ring of buffers; one is taken again only after its last copy has finished."""
    DEPTH, FLOATS = 8, 5 * 1024

    def __init__(self, device):
        self.device = device
        self.host = [torch.empty(self.FLOATS, dtype=torch.float32, pin_memory=True) for _ in range(self.DEPTH)]
        self.done = [None] * self.DEPTH
        self.turn = 0

    def upload(self, values: np.ndarray) -> torch.Tensor:
        if values.size > self.FLOATS:
            return torch.from_numpy(values).to(self.device)
        self.turn = (self.turn + 1) % self.DEPTH
        if self.done[self.turn] is None:
            self.done[self.turn] = torch.cuda.Event()
        else:
            self.done[self.turn].synchronize()
        staged = self.host[self.turn][:values.size].view(values.shape)
        staged.copy_(torch.from_numpy(values))
        out = torch.empty(values.shape, dtype=torch.float32, device=self.device)
        out.copy_(staged, non_blocking=True)
        self.done[self.turn].record()
        return out


_staging = {}


def _to_device(values: np.ndarray, device) -> torch.Tensor:
    if device.type != "cuda":
        return torch.from_numpy(values).to(device)
    if device not in _staging:
        _staging[device] = _Staging(device)
    return _staging[device].upload(values)


def sample_rows_on_device(logits: torch.Tensor, samplers: Sequence[Sampler]) -> torch.Tensor:
    """Row i of `logits` (float32 [n, vocab], on the device) is sampled with samplers[i]; the tokens stay on the
    device (int32 [n]) and nothing waits for them.  A sampler draws one uniform number per call unless it is greedy.
    Rows of one kind (arg max; the plain softmax; top-k or top-p) go through that kind's kernels together; where
    kinds are mixed, each kind's rows are gathered first."""
    n, vocab = logits.shape
    if n != len(samplers):
        raise ValueError(f"{n} rows of logits for {len(samplers)} samplers")
    dev = logits.device
    out = torch.empty(n, dtype=torch.int32, device=dev)
    kinds = [s.kind for s in samplers]
    if all(k == "greedy" for k in kinds):
        return ops.argmax(logits, out)
    # One copy to the device for everything the rows' kernels need, rows grouped by kind: temperature, uniform number,
    # top-p, top-k, and the row in `logits`.
    order = sorted(range(n), key=lambda i: _KIND_ORDER[kinds[i]])
    host = np.zeros((5, n), dtype=np.float32)
    ints = host.view(np.int32)
    for col, i in enumerate(order):
        s = samplers[i]
        if s.kind != "greedy":
            host[0, col], host[1, col], host[2, col] = s.temperature, s.next_uniform(), s.config.top_p
            ints[3, col] = s.config.top_k if 0 < s.config.top_k < vocab else 0
        ints[4, col] = i
    params = _to_device(host, dev)
    sorted_kinds = [kinds[i] for i in order]
    start = 0
    while start < n:
        kind = sorted_kinds[start]
        stop = start + sorted_kinds.count(kind)
        whole = stop - start == n                                 # then the rows are in their own order
        where = None if whole else params[4, start:stop].view(torch.int32).long()
        rows = logits if whole else logits.index_select(0, where)
        res = out if whole else torch.empty(stop - start, dtype=torch.int32, device=dev)
        if kind == "greedy":
            ops.argmax(rows, res)
        elif kind == "plain":
            ops.sample_temperature(rows, params[0, start:stop], params[1, start:stop], res)
        else:
            ops.sample_filtered(rows, params[0, start:stop], params[3, start:stop].view(torch.int32), params[2, start:stop],
                                params[1, start:stop], res)
        if not whole:
            out.index_copy_(0, where, res)
        start = stop
    return out


def sample_rows(logits: torch.Tensor, samplers: Sequence[Sampler]) -> List[int]:
    """`sample_rows_on_device`, with the tokens brought to the host."""
    return sample_rows_on_device(logits, samplers).tolist()
