"""bin/trace_run as a user runs it: a child process fed steps on its standard input, one at a time,
each sent only after the previous `done` line; the logits it writes are compared with the plain
implementation for the same requests replayed whole, with the last 32 tokens one by one, in
portions of changing size, and mixed with other requests on so few pages that they are used again."""
import json
import random
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

import traces
from model_folders import CONFIGS, assert_within_bfloat16_noise, relative_error, write_model
from plain_llama import PlainLlama

pytestmark = pytest.mark.gpu
ROOT = Path(__file__).resolve().parent.parent


def run_trace(model, dtype, steps, out, max_tokens, extra=()):
    cmd = [str(ROOT / "bin" / "trace_run"), "--model", str(model), "--dtype", dtype, "--out", str(out), "--max-tokens", str(max_tokens), *extra]
    proc = subprocess.Popen(cmd, stdin=subprocess.PIPE, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True)
    try:
        for s in steps:
            proc.stdin.write(json.dumps(s) + "\n")
            proc.stdin.flush()
            line = proc.stdout.readline().strip()
            assert line == f"done {s['step']}", (line, proc.stderr.read() if proc.poll() is not None else "")
        proc.stdin.close()
        assert proc.wait(timeout=60) == 0, proc.stderr.read()
    finally:
        if proc.poll() is None:
            proc.kill()
    got, vocab = {}, json.loads((Path(model) / "config.json").read_text())["vocab_size"]
    for step, rows in traces.wanted_positions(steps).items():
        data = np.fromfile(Path(out) / f"{step}.f32", dtype="<f4").reshape(len(rows), vocab)
        for key, row in zip(rows, data):
            got[key] = torch.from_numpy(row.copy())
    assert not [p for p in Path(out).glob("*.f32") if int(p.stem) not in traces.wanted_positions(steps)]
    return got


@pytest.fixture(scope="module")
def case(tmp_path_factory):
    folder = tmp_path_factory.mktemp("replayB")
    write_model(folder, CONFIGS["B"], seed=77)
    rng = random.Random(6)
    requests = {f"q{i}": [rng.randrange(384) for _ in range(n)] for i, n in enumerate([70, 1, 33, 129, 40, 9])}
    plain, rounded = PlainLlama(folder), PlainLlama(folder, storage=torch.bfloat16)
    want = {"float32": {r: plain.logits(t) for r, t in requests.items()}, "bfloat16": {r: rounded.logits(t) for r, t in requests.items()}}
    return folder, requests, want


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("mode", ["whole", "tail_singly", "portions", "mixed"])
def test_replay(case, tmp_path, dtype, mode):
    folder, requests, want = case
    steps = {"whole": traces.whole, "tail_singly": lambda r: traces.tail_singly(r, 32), "portions": traces.portions,
             "mixed": lambda r: traces.mixed(r, seed=12)}[mode](requests)
    if mode == "whole":                                              # logits asked for at some places only, and at none in one step
        steps = traces.whole(requests, want_every=3)
        steps[1]["entries"][0]["want"] = []
    got = run_trace(folder, dtype, steps, tmp_path / "out", traces.peak_tokens(steps, 64))
    if dtype == "float32":
        worst = max(relative_error(row, want[dtype][rid][pos]) for (rid, pos), row in got.items())
        assert worst < 2e-5, worst
    else:
        assert_within_bfloat16_noise(got, lambda k: want["float32"][k[0]][k[1]], lambda k: want["bfloat16"][k[0]][k[1]], mode)
    assert len(got) == sum(len(v) for v in traces.wanted_positions(steps).values())


def test_replay_needs_no_setup_and_says_what_is_wrong(case, tmp_path):
    folder, requests, _ = case
    bad = subprocess.run([str(ROOT / "bin" / "trace_run"), "--model", str(tmp_path / "nowhere"), "--dtype", "float32", "--out", str(tmp_path / "o"),
                          "--max-tokens", "64"], input="", capture_output=True, text=True)
    assert bad.returncode != 0 and "config.json" in bad.stderr
    usage = subprocess.run([str(ROOT / "bin" / "trace_run"), "--model", str(folder), "--dtype", "float16", "--out", str(tmp_path / "o"),
                            "--max-tokens", "64"], input="", capture_output=True, text=True)
    assert usage.returncode == 2 and "invalid choice" in usage.stderr
    empty = subprocess.run([str(ROOT / "bin" / "trace_run"), "--model", str(folder), "--dtype", "float32", "--out", str(tmp_path / "o"),
                            "--max-tokens", "64"], input="", capture_output=True, text=True)
    assert empty.returncode == 0 and empty.stdout == ""
