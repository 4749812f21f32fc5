"""The single-request loop: a prompt goes in, tokens come out one by one.

As the reference's `generate()` (src/runtime/generator.cpp:10-78): all prompt tokens but the
last run through the step function without logits (in portions of at most `prefill_rows`); the
last prompt token and every later token run singly and return the logits from which the next
token is sampled.  `max_positions` bounds prompt plus generated tokens (0 = the context length).
An end token is kept as the last generated token and stops the loop.
"""
from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Callable, Iterable, List, Optional, Sequence

from ..sampling import Sampler
from .runner import Runner, StepEntry


@dataclass
class GenerateResult:
    prompt_tokens: List[int]
    generated_tokens: List[int] = field(default_factory=list)
    stopped_by_end_token: bool = False
    prefill_ms: float = 0.0          # the prompt, including the sampling of the first new token
    decode_ms: float = 0.0
    decode_steps: int = 0


def generate(runner: Runner, sampler: Sampler, prompt_tokens: Sequence[int], max_positions: int = 0,
             end_tokens: Iterable[int] = (), on_token: Optional[Callable[[int], None]] = None,
             prefill_rows: Optional[int] = None, request="generate", sample=None) -> GenerateResult:
    """`sample(logits_row, sampler) -> token` replaces the sampler's own device sampling (tests without a GPU use it)."""
    prompt = [int(t) for t in prompt_tokens]
    if not prompt:
        raise ValueError("generate: prompt has no tokens")
    context = runner.max_positions
    if len(prompt) > context:
        raise ValueError(f"generate: prompt of {len(prompt)} tokens does not fit in the context length {context}")
    steps = context if max_positions <= 0 else min(max_positions, context)
    end_tokens = set(int(t) for t in end_tokens)
    chunk = min(prefill_rows or runner.max_rows, runner.max_rows)
    result = GenerateResult(prompt_tokens=prompt)

    runner.open(request)
    try:
        pos = 0
        batched = min(len(prompt) - 1, steps)
        t_start = t_first = time.perf_counter()
        while pos < batched:
            n = min(chunk, batched - pos)
            runner.step([StepEntry(request, prompt[pos:pos + n], ())])
            pos += n
        token = prompt[pos] if pos < len(prompt) else None
        while pos < steps:
            logits = runner.step([StepEntry(request, [token], (0,))])
            nxt = sampler.sample(logits[0]) if sample is None else sample(logits[0], sampler)     # the token reaches the host: the step has finished
            result.generated_tokens.append(nxt)
            if len(result.generated_tokens) == 1:
                t_first = time.perf_counter()
                result.prefill_ms = (t_first - t_start) * 1e3
            else:
                result.decode_steps += 1
            pos += 1
            if nxt in end_tokens:
                result.stopped_by_end_token = True
                break
            if on_token is not None:
                on_token(nxt)
            token = nxt
        if result.generated_tokens:
            result.decode_ms = (time.perf_counter() - t_first) * 1e3
    finally:
        runner.close(request)
    return result
