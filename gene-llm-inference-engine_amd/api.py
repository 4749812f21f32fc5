"""The Python entry point: a model folder in, tokens out.

    import geneinfer_amd as gi
    llm = gi.LLM("model_dir", dtype="bfloat16")
    out = llm.generate([1, 2, 3], steps=64, temperature=0.0)          # one request
    outs = llm.generate_many([[1, 2], [3, 4, 5]], steps=64)            # continuous batching

Option names follow the reference's command line (tools/generate_main.cpp:9-27): `steps` is the
most positions of prompt plus generated tokens, temperature 0 is greedy, top_k 0 and top_p 1 are off.
"""
from __future__ import annotations

import json
import time
from pathlib import Path
from typing import Iterable, List, Optional, Sequence

import torch

from .kernels import ops
from .engine import Engine, EngineConfig, EngineRequest, Runner, generate, load_model, random_model
from .sampling import Sampler, SamplerConfig


def end_tokens_of(folder) -> List[int]:
    """`eos_token_id` of the folder's config.json (a number or a list), else none."""
    try:
        eos = json.loads((Path(folder) / "config.json").read_text()).get("eos_token_id")
    except (OSError, ValueError):
        return []
    if isinstance(eos, int):
        return [eos]
    if isinstance(eos, list):
        return [int(t) for t in eos if isinstance(t, int)]
    return []


class LLM:
    """A loaded model with its cache and step function.

    max_seq_len  caps the context length (0 = the model's)
    page_size    positions per cache page
    max_tokens   positions the cache holds in all (0 = max_running full contexts, at most 65536 each)
    """

    def __init__(self, model, dtype="bfloat16", device="cuda:0", max_seq_len: int = 0, page_size: int = 16,
                 max_tokens: int = 0, max_running: int = 8, max_rows: int = 4096, end_tokens: Optional[Iterable[int]] = None):
        if isinstance(model, (str, Path)):
            self.model = load_model(model, dtype, device)
            self.end_tokens = list(end_tokens_of(model) if end_tokens is None else end_tokens)
        else:
            self.model = model
            self.end_tokens = list(end_tokens or [])
        limit = self.model.spec.max_positions
        context = min(max_seq_len, limit) if max_seq_len > 0 else limit
        max_tokens = max_tokens or max_running * min(context, 65536)
        self.runner = Runner(self.model, page_size=page_size, max_tokens=max_tokens, max_requests=max_running,
                             max_rows=max_rows, max_positions=context)

    def set_profiling(self, on: bool) -> None:
        """Per-kernel timing of everything this process steps from now on (`kernels.ops.KernelProfile`): the device
        is waited for around every kernel and no step is replayed from a captured graph, so the run is slower
        than an unobserved one.  `profile_report` gives the table; switching off forgets it."""
        self._profile = ops.set_profiling(on)
        self._profile_from = (self.runner.rows_run, self.runner.steps_run, time.perf_counter())

    def profile_report(self) -> str:
        """Empty if nothing was measured (the reference's `profile_report`, src/model/model.h:43-44)."""
        if getattr(self, "_profile", None) is None:
            return ""
        torch.cuda.synchronize()
        rows, steps, since = self._profile_from
        return self._profile.report(self.runner.rows_run - rows, self.runner.steps_run - steps, time.perf_counter() - since)

    def generate(self, prompt_ids: Sequence[int], steps: int = 0, temperature: float = 0.8, top_k: int = 0, top_p: float = 1.0,
                 seed: int = 1, on_token=None):
        sampler = Sampler(SamplerConfig(temperature, top_k, top_p, seed), self.model.spec.vocab_size)
        return generate(self.runner, sampler, prompt_ids, steps, self.end_tokens, on_token)

    def engine(self, config: Optional[EngineConfig] = None) -> Engine:
        return Engine(self.runner, config, self.end_tokens)

    def generate_many(self, prompts: Sequence[Sequence[int]], steps: int = 0, temperature: float = 0.8, top_k: int = 0,
                      top_p: float = 1.0, seed: int = 1, config: Optional[EngineConfig] = None):
        """Every prompt as a request of its own through the scheduler; request i samples with seed + i."""
        eng = self.engine(config)
        ids = [eng.submit(EngineRequest(p, steps, SamplerConfig(temperature, top_k, top_p, seed + i))) for i, p in enumerate(prompts)]
        eng.run_until_idle()
        return [eng.result(i) for i in ids]
