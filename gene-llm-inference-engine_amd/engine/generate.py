"""The single-request loop: a prompt goes in, tokens come out one by one.

As the reference's `generate()` (src/runtime/generator.cpp:10-78): all prompt tokens but the
last run through the step function without logits (in portions of at most `prefill_rows`); the
last prompt token and every later token run singly and return the logits from which the next
token is sampled.  Where the runner can take a step's token from the device (and the sampler draws
there), the next step is put in the queue before the host has read the token, so the device does
not wait for the host between tokens; an end token then costs one step whose result nobody sees.  `max_positions` bounds prompt plus generated tokens (0 = the context length).
An end token is kept as the last generated token and stops the loop.
"""
from __future__ import annotations

import time
from dataclasses import dataclass, field
from typing import Callable, Iterable, List, Optional, Sequence

from ..sampling import Sampler, sample_rows_on_device
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
        ahead = sample is None and pos < steps and getattr(runner, "can_step_from_device", False) and runner.model.device.type == "cuda"

        def took(nxt) -> bool:
            """Books for one generated token; False when it ends the request."""
            nonlocal t_first
            result.generated_tokens.append(nxt)
            if len(result.generated_tokens) == 1:
                t_first = time.perf_counter()
                result.prefill_ms = (t_first - t_start) * 1e3
            else:
                result.decode_steps += 1
            if nxt in end_tokens:
                result.stopped_by_end_token = True
                return False
            if on_token is not None:
                on_token(nxt)
            return True

        if ahead:
            import torch
            landing, landed = torch.empty(1, dtype=torch.int32, pin_memory=True), torch.cuda.Event()
            logits = runner.step([StepEntry(request, [token], (0,))])
            while True:
                on_device = sample_rows_on_device(logits, [sampler])
                landing.copy_(on_device, non_blocking=True)
                landed.record()
                pos += 1
                if pos < steps:                               # the next step is queued before the host knows its token
                    logits = runner.step_from_device([request], on_device)
                landed.synchronize()
                if not took(int(landing[0])) or pos >= steps:
                    break
        else:
            while pos < steps:
                logits = runner.step([StepEntry(request, [token], (0,))])
                nxt = sampler.sample(logits[0]) if sample is None else sample(logits[0], sampler)     # the token reaches the host: the step has finished
                pos += 1
                if not took(nxt):
                    break
                token = nxt
        if result.generated_tokens:
            result.decode_ms = (time.perf_counter() - t_first) * 1e3
    finally:
        runner.close(request)
    return result
