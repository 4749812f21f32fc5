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
                            "--no-echo", "--quiet", "--profile"], capture_output=True, text=True, timeout=170)
    assert again.stdout == quiet.stdout                                         # the same seed, the same tokens, watched or not
    assert "device profile: 6 positions in 5 steps" in again.stderr and "gemm_bf16" in again.stderr and "weights GB/s" in again.stderr


@pytest.mark.gpu
def test_gi_generate_from_a_configuration_alone_draws_the_weights_make_random_model_writes(tmp_path):
    """--config FILE --random-seed S: no folder; the tokens are those of the folder that make_random_model writes for the same seed."""
    cfg = tmp_path / "config.json"
    cfg.write_text(json.dumps(full_config(CONFIGS["B"])))
    made = subprocess.run([str(ROOT / "bin" / "make_random_model"), "--config", str(cfg), "--out", str(tmp_path / "m"), "--seed", "4", "--dtype", "float32"],
                          capture_output=True, text=True, timeout=120)
    assert made.returncode == 0, made.stderr
    common = ["--prompt-ids", "5 9 200 31", "--steps", "12", "--temperature", "0", "--weights", "f32", "--no-echo", "--quiet"]
    a = subprocess.run([str(ROOT / "bin" / "gi_generate"), "--config", str(cfg), "--random-seed", "4", *common], capture_output=True, text=True, timeout=170)
    b = subprocess.run([str(ROOT / "bin" / "gi_generate"), "--model", str(tmp_path / "m"), *common], capture_output=True, text=True, timeout=170)
    assert a.returncode == 0 and b.returncode == 0, a.stderr + b.stderr
    assert len(a.stdout.split()) == 9 and a.stdout == b.stdout


def test_gi_generate_usage_errors(tmp_path):
    exe = str(ROOT / "bin" / "gi_generate")
    for args, msg in (([], "give --model DIR, or --config FILE"), (["--model", "x", "--config", "y"], "give --model DIR, or --config FILE"),
                      (["--model", "x", "--weights", "int8"], "--weights must be native or f32"),
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
    assert int(rows[0][7]) == 0 and int(rows[1][7]) == 0                        # cached positions of the measured run
    warm = subprocess.run(common + ["--warm-cache"], capture_output=True, text=True, timeout=170)
    assert warm.returncode == 0, warm.stdout + warm.stderr
    rows = [line.split() for line in warm.stdout.splitlines() if line[:1].isdigit()]
    assert int(rows[0][7]) == 48 and int(rows[1][7]) == 4 * 48
    off = subprocess.run(common + ["--no-prefix-cache", "--profile"], capture_output=True, text=True, timeout=170)
    assert "device profile: " in off.stdout and "gemm_exact" in off.stdout
    assert off.returncode == 0 and all(int(line.split()[7]) == 0 for line in off.stdout.splitlines() if line[:1].isdigit())


@pytest.mark.gpu
def test_benches_take_a_configuration_alone_and_requests_of_their_own_lengths(tmp_path):
    """--config FILE: random weights drawn on the device, no folder.  gi_serve_bench with lengths LO:HI and a row budget: in
    32-bit every request still generates what it generates alone, with steps of at most --step-rows rows."""
    from model_folders import full_config
    cfg = tmp_path / "config.json"
    cfg.write_text(json.dumps(full_config(CONFIGS["B"])))
    r = subprocess.run([str(ROOT / "bin" / "gi_serve_bench"), "--config", str(cfg), "--random-seed", "3", "--concurrency", "2,4", "--prompt-tokens", "5:60",
                        "--decode-tokens", "3:14", "--runs", "1", "--weights", "f32", "--block-size", "8", "--step-rows", "24"],
                       capture_output=True, text=True, timeout=170)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "prompt 5 to 60 + decode 3 to 14 tokens per request" in r.stdout and "max rows per pass 24" in r.stdout and "random weights (seed 3)" in r.stdout
    rows = [line.split() for line in r.stdout.splitlines() if line[:1].isdigit()]
    assert [int(row[0]) for row in rows] == [2, 4] and all("identical" in " ".join(row) for row in rows) and all(float(row[5]) <= 24 for row in rows)
    quick = subprocess.run([str(ROOT / "bin" / "gi_serve_bench"), "--config", str(cfg), "--concurrency", "3", "--runs", "1", "--no-compare"],
                           capture_output=True, text=True, timeout=170)
    assert quick.returncode == 0 and "not compared" in quick.stdout, quick.stdout + quick.stderr
    drawn = subprocess.run([str(ROOT / "bin" / "gi_serve_bench"), "--config", str(cfg), "--concurrency", "3", "--runs", "1", "--weights", "f32",
                            "--temperature", "0.8", "--top-k", "5", "--top-p", "0.9", "--seed", "4"], capture_output=True, text=True, timeout=170)
    assert drawn.returncode == 0 and "temperature 0.8, top-k 5, top-p 0.9" in drawn.stdout and "identical to running alone" in drawn.stdout, drawn.stdout + drawn.stderr
    one = subprocess.run([str(ROOT / "bin" / "gi_bench"), "--config", str(cfg), "--prompt-tokens", "20", "--decode-tokens", "5", "--runs", "1"],
                         capture_output=True, text=True, timeout=170)
    assert one.returncode == 0 and "workload: 20 prompt + 5 decode positions" in one.stdout and "random weights (seed 0)" in one.stdout, one.stdout + one.stderr


def test_gi_serve_bench_usage_errors():
    exe = str(ROOT / "bin" / "gi_serve_bench")
    for args, msg in (([], "give --model DIR, or --config FILE"), (["--model", "x", "--prompt-tokens", "9:3"], "LO not above HI"),
                      (["--model", "x", "--config", "y"], "give --model DIR, or --config FILE"), (["--model", "x", "--concurrency", "0"], "--concurrency needs positive integers"),
                      (["--model", "x", "--weights", "int8"], "--weights must be native or f32"), (["--model", "x", "--runs"], "missing value for --runs"), (["--model", "x", "--top-p", "2"], "--top-p must be in (0, 1]"),
                      (["--model", "x", "--temperature", "hot"], "invalid number for --temperature"),
                      (["--model", "x", "--max-seq-len", "8"], "--max-seq-len is shorter"), (["--model", "x", "--what"], "unknown option --what")):
        r = subprocess.run([exe, *args], capture_output=True, text=True, timeout=60)
        assert r.returncode == 2 and msg in r.stderr and "usage: gi_serve_bench" in r.stderr


@pytest.mark.gpu
def test_gi_bench_reports_one_request(tmp_path):
    write_model(tmp_path / "m", CONFIGS["A"], seed=2)
    report = tmp_path / "report.json"
    r = subprocess.run([str(ROOT / "bin" / "gi_bench"), "--model", str(tmp_path / "m"), "--prompt-tokens", "20", "--decode-tokens", "9", "--runs", "2",
                        "--label", "tiny", "--json", str(report), "--block-size", "4", "--profile"], capture_output=True, text=True, timeout=170)
    assert r.returncode == 0, r.stderr
    assert "device profile: 29 positions in 10 steps" in r.stdout                # one more run, the watched one, after the measured two
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
    for args, msg in (([], "give --model DIR, or --config FILE"), (["--model", "x", "--runs", "0"], "must be positive"),
                      (["--model", "x", "--weights", "int8"], "--weights must be native or f32"), (["--model", "x", "--isa", "avx2"], "unknown option --isa")):
        r = subprocess.run([exe, *args], capture_output=True, text=True, timeout=60)
        assert r.returncode == 2 and msg in r.stderr and "usage: gi_bench" in r.stderr


@pytest.mark.gpu
def test_gi_forward_dumps_logits_and_the_last_position_layer_by_layer(tmp_path):
    import numpy as np
    from plain_llama import read_model_folder
    name = "B"
    write_model(tmp_path / "m", CONFIGS[name], seed=6)
    cfg, vocab, hidden = CONFIGS[name], CONFIGS[name]["vocab_size"], CONFIGS[name]["hidden_size"]
    tokens = [3, 14, 15, 92, 65, 35, 89, 79, 32, 38, 46, 26, 43, 38, 32, 79, 50, 28, 84, 19]
    exe = str(ROOT / "bin" / "gi_forward")
    ids = [str(t) for t in tokens]
    r = subprocess.run([exe, str(tmp_path / "m"), str(tmp_path / "one"), "--weights", "f32", "--block-size", "4", *ids], capture_output=True, text=True, timeout=170)
    assert r.returncode == 0 and f"positions={len(tokens)} vocab={vocab} avg_ms_per_token=" in r.stdout, r.stdout + r.stderr
    logits = torch.from_numpy(np.fromfile(tmp_path / "one" / "logits.f32", dtype="<f4")).reshape(len(tokens), vocab)
    want = PlainLlama(tmp_path / "m").logits(tokens)
    assert float((logits.double() - want).abs().max() / want.abs().max()) < 2e-5
    _, weights = read_model_folder(tmp_path / "m")
    embedding = torch.from_numpy(np.fromfile(tmp_path / "one" / "embedding.f32", dtype="<f4"))
    assert torch.equal(embedding, weights["model.embed_tokens.weight"][tokens[-1]].float())       # of the last position
    files = sorted(p.name for p in (tmp_path / "one").glob("layer*.f32"))
    assert files == sorted(f"layer{i:02d}_{tag}.f32" for i in range(cfg["num_hidden_layers"]) for tag in ("attn_out", "ffn_out"))
    assert all((tmp_path / "one" / f).stat().st_size == 4 * hidden for f in files)
    final = torch.from_numpy(np.fromfile(tmp_path / "one" / "final_norm.f32", dtype="<f4"))
    head = weights.get("lm_head.weight", weights["model.embed_tokens.weight"]).float()
    assert float((head @ final - logits[-1]).abs().max() / logits[-1].abs().max()) < 1e-5            # what the logits are taken from
    # a portion on top of single tokens, cut by --max-batch, after a decoy sequence that is rewound: the same rows, bit for bit
    r = subprocess.run([exe, str(tmp_path / "m"), str(tmp_path / "two"), "--weights", "f32", "--block-size", "4", "--prefill", "12", "--head", "5",
                        "--max-batch", "4", "--decoy", *ids], capture_output=True, text=True, timeout=170)
    assert r.returncode == 0, r.stderr
    rows = torch.from_numpy(np.fromfile(tmp_path / "two" / "logits.f32", dtype="<f4")).reshape(-1, vocab)
    assert rows.shape[0] == len(tokens) - 11 and torch.equal(rows, logits[11:])
    assert not list((tmp_path / "two").glob("layer*.f32")) and not (tmp_path / "two" / "embedding.f32").exists()
    # --traced: the whole sequence as portions with the trace on: the last position's activations are those of the token-by-token run
    r = subprocess.run([exe, str(tmp_path / "m"), str(tmp_path / "four"), "--weights", "f32", "--block-size", "4", "--prefill", "20", "--max-batch", "7",
                        "--traced", *ids], capture_output=True, text=True, timeout=170)
    assert r.returncode == 0, r.stderr
    assert np.array_equal(np.fromfile(tmp_path / "four" / "logits.f32", dtype="<f4"), logits[-1].numpy())
    for f in files + ["embedding.f32", "final_norm.f32"]:
        assert np.array_equal(np.fromfile(tmp_path / "four" / f, dtype="<f4"), np.fromfile(tmp_path / "one" / f, dtype="<f4")), f
    # --pos-shift: a portion anywhere but where the cache ends is refused with a clean error (tests/verify_batch.py:128-139,
    # tests/verify_device.py:233-235 of the reference ask the same of it)
    for extra, msg in ((["--prefill", "3", "--head", "1", "--pos-shift", "1"], "leaves a gap"),
                       (["--max-seq-len", "20", "--prefill", "20", "--pos-shift", "1"], "exceed the context length 20"),
                       (["--prefill", "4", "--head", "2", "--pos-shift", "-1"], "lies under")):
        r = subprocess.run([exe, str(tmp_path / "m"), str(tmp_path / "five"), "--weights", "f32", *extra, *ids], capture_output=True, text=True, timeout=170)
        assert r.returncode == 1 and msg in r.stderr, (extra, r.stderr)
    native = subprocess.run([exe, str(tmp_path / "m"), str(tmp_path / "three"), "--prefill", "20", *ids], capture_output=True, text=True, timeout=170)
    assert native.returncode == 0 and (tmp_path / "three" / "logits.f32").stat().st_size == 4 * vocab


def test_gi_forward_usage_and_errors(tmp_path):
    exe = str(ROOT / "bin" / "gi_forward")
    r = subprocess.run([exe, "x"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 2 and "usage: gi_forward" in r.stderr
    for args, msg in ((["x", str(tmp_path / "o")], "no token ids given"), (["x", str(tmp_path / "o"), "--prefill", "3", "--head", "3", "1", "2", "3"], "--head must be smaller"),
                      (["x", str(tmp_path / "o"), "--prefill", "9", "1", "2"], "--prefill must be between"), (["x", str(tmp_path / "o"), "--prefill"], "--prefill needs a value")):
        r = subprocess.run([exe, *args, *([] if "1" in args or "--prefill" == args[-1] else ["--max-seq-len", "8"])], capture_output=True, text=True, timeout=60)
        assert r.returncode == 1 and msg in r.stderr, r.stderr
