"""The command line: bin/gi_generate with the reference's options, bin/make_random_model."""
import json
import subprocess
import sys
from pathlib import Path

import pytest
import torch

from model_folders import CONFIGS, full_config, write_model
from plain_llama import PlainLlama

ROOT = Path(__file__).resolve().parent.parent


@pytest.mark.gpu
def test_gi_generate_greedy_dumps_the_plain_tokens(tmp_path):
    write_model(tmp_path / "m", CONFIGS["A"], seed=9)
    prompt = [17, 4, 200, 33, 91]
    dump = tmp_path / "tokens.txt"
    r = subprocess.run([str(ROOT / "bin" / "gi_generate"), "--model", str(tmp_path / "m"), "--prompt-ids", " ".join(map(str, prompt)),
                        "--steps", str(len(prompt) + 7), "--temperature", "0", "--weights", "f32", "--dump-tokens", str(dump), "--page-size", "4"],
                       capture_output=True, text=True, timeout=170)
    assert r.returncode == 0, r.stderr
    lines = dump.read_text().splitlines()
    want = PlainLlama(tmp_path / "m").greedy(prompt, 8)
    assert [int(t) for t in lines[0].split()] == prompt and [int(t) for t in lines[1].split()] == want
    assert r.stdout.split() == [str(t) for t in prompt + want]                 # echo of the prompt, then the tokens as they come
    assert "prompt: 5 tokens" in r.stderr and "generated: 8 tokens" in r.stderr and "temperature 0.00" in r.stderr
    quiet = subprocess.run([str(ROOT / "bin" / "gi_generate"), "--model", str(tmp_path / "m"), "--prompt-ids", "1,2,3", "--steps", "6", "--seed", "5",
                            "--no-echo", "--quiet"], capture_output=True, text=True, timeout=170)
    assert quiet.returncode == 0 and len(quiet.stdout.split()) == 4 and "prompt:" not in quiet.stderr and "gpu:" not in quiet.stderr
    again = subprocess.run([str(ROOT / "bin" / "gi_generate"), "--model", str(tmp_path / "m"), "--prompt-ids", "1,2,3", "--steps", "6", "--seed", "5",
                            "--no-echo", "--quiet"], capture_output=True, text=True, timeout=170)
    assert again.stdout == quiet.stdout                                         # the same seed, the same tokens


def test_gi_generate_usage_errors(tmp_path):
    exe = str(ROOT / "bin" / "gi_generate")
    for args, msg in (([], "--model is required"), (["--model", "x", "--weights", "int8"], "--weights must be native or f32"),
                      (["--model", "x", "--frobnicate"], "unknown option --frobnicate"), (["--model"], "missing value for --model"),
                      (["--model", "x", "--steps", "ten"], "invalid integer for --steps"), (["--model", "x", "--device", "cpu"], "only gpu exists")):
        r = subprocess.run([exe, *args], capture_output=True, text=True, timeout=60)
        assert r.returncode == 2 and msg in r.stderr and "usage: gi_generate" in r.stderr
    r = subprocess.run([exe, "--model", str(tmp_path), "--prompt-ids", "1"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 1 and r.stderr.startswith("error:")                  # no config.json there


def test_make_random_model_writes_a_loadable_folder(tmp_path):
    cfg = tmp_path / "config.json"
    cfg.write_text(json.dumps(full_config(CONFIGS["C"])))
    r = subprocess.run([str(ROOT / "bin" / "make_random_model"), "--config", str(cfg), "--out", str(tmp_path / "m"), "--seed", "3", "--dtype", "float32"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    logits = PlainLlama(tmp_path / "m").logits([1, 2, 3])
    assert logits.shape == (3, 301) and torch.isfinite(logits).all()


@pytest.mark.gpu
def test_gi_serve_bench_levels_generate_what_each_request_generates_alone(tmp_path):
    """In 32-bit the tokens do not depend on who else runs.  Requests admitted together find nothing in an
    empty index (the pages are named once they are full); with --warm-cache the unmeasured run has left every
    prompt's full pages (block size 8, 50 prompt tokens of which the last is always computed: 6 pages)."""
    write_model(tmp_path / "m", CONFIGS["B"], seed=4)
    exe = str(ROOT / "bin" / "gi_serve_bench")
    common = [exe, "--model", str(tmp_path / "m"), "--concurrency", "1,4", "--prompt-tokens", "50", "--decode-tokens", "12", "--runs", "1",
              "--weights", "f32", "--block-size", "8", "--shared-prefix", "40"]
    r = subprocess.run(common, capture_output=True, text=True, timeout=170)
    assert r.returncode == 0, r.stdout + r.stderr
    rows = [line.split() for line in r.stdout.splitlines() if line[:1].isdigit()]
    assert [int(row[0]) for row in rows] == [1, 4] and all("identical" in " ".join(row) for row in rows)
    assert int(rows[0][6]) == 0 and int(rows[1][6]) == 0                        # cached positions of the measured run
    warm = subprocess.run(common + ["--warm-cache"], capture_output=True, text=True, timeout=170)
    assert warm.returncode == 0, warm.stdout + warm.stderr
    rows = [line.split() for line in warm.stdout.splitlines() if line[:1].isdigit()]
    assert int(rows[0][6]) == 48 and int(rows[1][6]) == 4 * 48
    off = subprocess.run(common + ["--no-prefix-cache"], capture_output=True, text=True, timeout=170)
    assert off.returncode == 0 and all(int(line.split()[6]) == 0 for line in off.stdout.splitlines() if line[:1].isdigit())


def test_gi_serve_bench_usage_errors():
    exe = str(ROOT / "bin" / "gi_serve_bench")
    for args, msg in (([], "--model is required"), (["--model", "x", "--concurrency", "0"], "--concurrency needs positive integers"),
                      (["--model", "x", "--weights", "int8"], "--weights must be native or f32"), (["--model", "x", "--runs"], "missing value for --runs"),
                      (["--model", "x", "--max-seq-len", "8"], "--max-seq-len is shorter"), (["--model", "x", "--what"], "unknown option --what")):
        r = subprocess.run([exe, *args], capture_output=True, text=True, timeout=60)
        assert r.returncode == 2 and msg in r.stderr and "usage: gi_serve_bench" in r.stderr


@pytest.mark.gpu
def test_gi_bench_reports_one_request(tmp_path):
    write_model(tmp_path / "m", CONFIGS["A"], seed=2)
    report = tmp_path / "report.json"
    r = subprocess.run([str(ROOT / "bin" / "gi_bench"), "--model", str(tmp_path / "m"), "--prompt-tokens", "20", "--decode-tokens", "9", "--runs", "2",
                        "--label", "tiny", "--json", str(report), "--block-size", "4"], capture_output=True, text=True, timeout=170)
    assert r.returncode == 0, r.stderr
    assert "workload: 20 prompt + 9 decode positions, 2 measured runs (+1 warmup)" in r.stdout and "| tiny |" in r.stdout
    j = json.loads(report.read_text())
    assert j["prompt_tokens"] == 20 and j["decode_tokens"] == 9 and j["label"] == "tiny" and j["bf16_weights"] is True
    assert j["prefill_tokens_per_s"] > 0 and j["decode_ms_min"] <= j["decode_ms_median"] <= j["decode_ms_p95"] <= j["decode_ms_max"]
    cfg = CONFIGS["A"]
    kv_dim = cfg["num_key_value_heads"] * (cfg.get("head_dim") or cfg["hidden_size"] // cfg["num_attention_heads"])
    assert j["cache_bytes_per_token"] == cfg["num_hidden_layers"] * 2 * kv_dim * 2 * (20 + 9 // 2)
    clamped = subprocess.run([str(ROOT / "bin" / "gi_bench"), "--model", str(tmp_path / "m"), "--prompt-tokens", "500", "--decode-tokens", "40", "--runs", "1",
                              "--max-seq-len", "32", "--weights", "f32", "--sequential-prefill"], capture_output=True, text=True, timeout=170)
    assert clamped.returncode == 0 and "workload: 31 prompt + 1 decode positions" in clamped.stdout, clamped.stdout + clamped.stderr


def test_gi_bench_usage_errors():
    exe = str(ROOT / "bin" / "gi_bench")
    for args, msg in (([], "--model is required"), (["--model", "x", "--runs", "0"], "must be positive"),
                      (["--model", "x", "--weights", "int8"], "--weights must be native or f32"), (["--model", "x", "--isa", "avx2"], "unknown option --isa")):
        r = subprocess.run([exe, *args], capture_output=True, text=True, timeout=60)
        assert r.returncode == 2 and msg in r.stderr and "usage: gi_bench" in r.stderr
