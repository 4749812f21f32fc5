"""A context of sixteen thousand positions in 32-bit: the softmax of a late row sums over more keys than any other test's
(a 32-bit running sum would lose digits there; the reference sums in 64-bit, src/kernels/kernels.cpp:95-100), the page table
of a request runs to over a thousand pages, and the prompt goes in as portions of 4,096 rows before single tokens follow."""
import random

import pytest
import torch

from model_folders import TINY_D, relative_error, write_model
from plain_llama import PlainLlama

pytestmark = pytest.mark.gpu
CONTEXT = 16384 + 64


def test_sixteen_thousand_positions_in_32_bit(tmp_path):
    from geneinfer_amd.engine import Runner, StepEntry, load_model
    sizes = dict(TINY_D, max_position_embeddings=CONTEXT, num_hidden_layers=1)
    write_model(tmp_path, sizes, seed=77)
    rng = random.Random(5)
    toks = [rng.randrange(sizes["vocab_size"]) for _ in range(16384 + 3)]
    prompt = 16384 - 5
    places = list(range(prompt - 2, len(toks)))               # the last rows of the last portion, then every single token
    want = PlainLlama(tmp_path).logits_at(toks, places)
    model = load_model(tmp_path, "float32", "cuda:0")
    runner = Runner(model, page_size=16, max_tokens=CONTEXT, max_requests=1, max_rows=4096)
    runner.open("r")
    got, fed = {}, 0
    while fed < prompt:
        n = min(4096, prompt - fed)
        wanted = [p - fed for p in places if fed <= p < fed + n]
        logits = runner.step([StepEntry("r", toks[fed:fed + n], tuple(wanted))])
        for w, row in zip(wanted, logits.cpu() if wanted else ()):
            got[fed + w] = row
        fed += n
    for p in range(prompt, len(toks)):
        got[p] = runner.step([StepEntry("r", [toks[p]], (0,))])[0].cpu()
    runner.close("r")
    assert sorted(got) == places
    worst = max(relative_error(got[p], want[i]) for i, p in enumerate(places))
    print(f"16,384 positions in float32: worst relative error {worst:.2e}")
    assert worst < 2e-5, f"worst relative error {worst:.3e}"
