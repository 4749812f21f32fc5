"""Decode and prefill throughput of the engine at the Llama-3.2-1B shape, random weights, one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--config FILE] [--prefill-tokens T] [--layers L] [--no-points]

A step is one decode step of the whole batch (default batch 8, each request on a 2,048-token
prompt in a 4,096-token context), through the scheduler with its defaults.  After W warm-up steps,
five windows of exactly K steps each are timed one after the other (5 K + W new tokens a request:
256 with the defaults, the benchmark's workload); `value` and `ms_per_step` are the median window's,
`ms_per_step_min` the fastest's.  Prints ONE JSON line: decoded tokens a second, the 2,048-token
prefill (median of 5), the decode step's roofline fraction against the published HBM peak and
against the read bandwidth a plain kernel of this library reaches on this chip, the prefill's
fraction against the published matrix peak and against a bare loop of matrix instructions, and decode
at batch 1 and 64 (medians of 5 windows as well).  --config FILE runs the same on another configuration of the
architecture (a config.json; `configs/` holds the Llama 3.2 3B and 3.1 8B shapes), --prefill-tokens T times a prompt of
another length.
"""
import argparse
import json
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

# MI355X published peaks
HBM_GBS = 8000.0
PEAK_TFLOPS = {"bf16": 2500.0, "fp32": 157.3}

LLAMA_1B = dict(hidden_size=2048, intermediate_size=8192, num_hidden_layers=16, num_attention_heads=32, num_key_value_heads=8,
                head_dim=64, vocab_size=128256, max_position_embeddings=4096, rope_theta=500000.0, rms_norm_eps=1e-5,
                tie_word_embeddings=True,
                rope_scaling=dict(rope_type="llama3", factor=32.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                  original_max_position_embeddings=8192))
PROMPT, NEW_TOKENS, CONTEXT, PAGE = 2048, 256, 4096, 16


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=48, help="decode steps per timed window (five windows are timed)")
    ap.add_argument("--warmup", type=int, default=16)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--dtype", choices=["bf16", "fp32"], default="bf16")
    ap.add_argument("--layers", type=int, default=0, help="fewer layers than the configuration has (0 = all); named in the record")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and batch 64 points")
    ap.add_argument("--config", default="", help="a config.json of another size of the architecture (default: the Llama-3.2-1B shape)")
    ap.add_argument("--prefill-tokens", type=int, default=PROMPT, help="length of the timed prompt")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU; --gpus {args.gpus} is not supported by this single-GPU engine")
        return 2

    import torch
    from geneinfer_amd.config import LlamaConfig
    from geneinfer_amd.engine import Engine, EngineConfig, EngineRequest, Runner, StepEntry, random_model
    from geneinfer_amd.kernels import ops
    from geneinfer_amd.sampling import Sampler, SamplerConfig, sample_rows

    sizes, name = dict(LLAMA_1B), "Llama-3.2-1B"
    if args.config:
        sizes, name = json.loads(Path(args.config).read_text()), Path(args.config).stem
    T = args.prefill_tokens
    context_len = max(CONTEXT, T + 64)
    sizes["max_position_embeddings"] = max(context_len, sizes.get("max_position_embeddings", 0))
    layers_full = sizes["num_hidden_layers"]
    if args.layers:
        sizes["num_hidden_layers"] = args.layers
    config = LlamaConfig.from_dict(sizes) if not args.config else __import__("geneinfer_amd.config", fromlist=["parse_config"]).parse_config(sizes)
    dtype = "bfloat16" if args.dtype == "bf16" else "float32"
    model = random_model(config, seed=0, dtype=dtype, device="cuda:0", draw_on_device=True)
    vocab = config.vocab_size
    gen = torch.Generator().manual_seed(1)

    WINDOWS, PREFILL_WARMUP = 5, 4

    def make_runner(batch, per_request=0):
        per_request = per_request or -(-(PROMPT + WINDOWS * args.steps + args.warmup + 2 * batch + 8) // 64) * 64
        return Runner(model, page_size=PAGE, max_tokens=batch * per_request, max_requests=batch, max_rows=max(PROMPT, T, batch),
                      max_positions=context_len)

    def prefill(runner, rid, toks):
        runner.open(rid)
        return runner.step([StepEntry(rid, toks, (T - 1,))])

    def decode(batch, steps, warmup):
        """Greedy decoding of `batch` requests after their prompts, through the scheduler as serving runs it (its
        defaults: prefix sharing on, decoding ahead); returns [(seconds for `steps` decode steps, mean context at the
        middle of them)] for WINDOWS windows timed one after the other, sorted by time."""
        runner = make_runner(batch)
        engine = Engine(runner, EngineConfig(max_running=batch))
        limit = min(CONTEXT, PROMPT + WINDOWS * steps + warmup + 2 * batch + 4)
        for r in range(batch):
            engine.submit(EngineRequest(torch.randint(0, vocab, (PROMPT,), generator=gen).tolist(), limit, SamplerConfig(temperature=0.0)))
        decoding = 0
        while decoding < 2:                                  # the prompts, in steps of up to max_rows rows, until steps hold decode rows only
            rows = engine.stats.rows
            assert engine.step()
            decoding = decoding + 1 if engine.stats.rows - rows == batch and engine.stats.passes > batch else 0
        for _ in range(warmup):
            engine.step()
        windows = []
        for _ in range(WINDOWS):
            torch.cuda.synchronize()
            context = sum(runner.length(job.key) for job in engine.running) / batch + steps / 2
            passes = engine.stats.passes
            t0 = time.perf_counter()
            for _ in range(steps):
                engine.step()
            torch.cuda.synchronize()
            windows.append((time.perf_counter() - t0, context))
            assert engine.stats.passes - passes == steps and len(engine.running) == batch, "a timed step was not a decode step of the whole batch"
        del engine, runner
        torch.cuda.empty_cache()
        return sorted(windows)

    # ---- prefill of one 2,048-token prompt (median of 5 after PREFILL_WARMUP untimed ones: the first few run some percent slower)
    runner = make_runner(1, T + 64)
    greedy = Sampler(SamplerConfig(temperature=0.0), vocab)
    times = []
    for i in range(PREFILL_WARMUP + 5):
        toks = torch.randint(0, vocab, (T,), generator=gen).tolist()            # the prompt is there before the clock starts
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        logits = prefill(runner, i, toks)
        sample_rows(logits, [greedy])          # the first token reaches the host, drawn as generation draws it
        times.append(time.perf_counter() - t0)
        runner.close(i)
    prefill_s = sorted(times[PREFILL_WARMUP:])[2]
    del runner
    torch.cuda.empty_cache()
    L, D, I, V = config.num_hidden_layers, config.hidden_size, config.intermediate_size, vocab
    A, KV, hd, H = config.attn_dim, config.kv_dim, config.head_dim, config.num_attention_heads
    layer_params = D * (A + 2 * KV) + A * D + 3 * I * D
    prefill_flops = 2.0 * L * layer_params * T + L * 4.0 * H * hd * T * (T + 1) / 2 + 2.0 * V * D
    prefill_rec = {"value": round(T / prefill_s, 1), "tokens": T, "ms": round(prefill_s * 1e3, 3),
                   "frac": round(prefill_flops / prefill_s / (PEAK_TFLOPS[args.dtype] * 1e12), 4)}

    # ---- what a plain kernel reads and a bare loop of matrix instructions computes on this chip
    own_gbs = ops.measured_read_bandwidth("cuda:0")
    own_tflops = ops.measured_mfma_rate("cuda:0") if args.dtype == "bf16" else None
    prefill_rec["tflops"] = round(prefill_flops / prefill_s / 1e12, 1)
    if own_tflops:
        prefill_rec["own_peak_tflops"], prefill_rec["frac_of_own_peak"] = round(own_tflops, 1), round(prefill_flops / prefill_s / 1e12 / own_tflops, 4)

    # ---- decode
    windows = decode(args.batch, args.steps, args.warmup)
    dt, context = windows[len(windows) // 2]
    elem = 2 if args.dtype == "bf16" else 4
    weight_bytes = model.weight_bytes_read_per_step()
    kv_bytes = args.batch * context * L * 2 * KV * elem
    achieved = (weight_bytes + kv_bytes) / (dt / args.steps) / 1e9
    points = {}
    if not args.no_points:
        for b in (1, 64):
            w = decode(b, max(8, args.steps // 2), 8)
            points[f"decode_b{b}"] = round(b * max(8, args.steps // 2) / w[len(w) // 2][0], 1)

    rec = {
        "metric": f"decode tok/s at batch 1/8/64 + prefill tok/s at {T:,} tokens, {name}",
        "value": round(args.batch * args.steps / dt, 1), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(dt / args.steps * 1e3, 4), "ms_per_step_min": round(windows[0][0] / args.steps * 1e3, 4), "windows": WINDOWS,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": args.dtype, "data": "synthetic: random weights N(0, 0.02) by a stated formula of seed, tensor name and index, uniform random token ids",
        "config": {"model": f"{name} shape", "layers": L, "layers_of_config": layers_full, "hidden": D, "heads": H,
                   "kv_heads": config.num_key_value_heads, "head_dim": hd, "intermediate": I, "vocab": V, "global_batch": args.batch,
                   "seq_len": context_len, "prompt_len": PROMPT, "decode_context": context, "page_size": PAGE, "tied_embeddings": bool(sizes.get("tie_word_embeddings", False)),
                   "rope": f"{(sizes.get('rope_scaling') or {}).get('rope_type', 'plain')} theta {sizes.get('rope_theta', 10000.0):g} factor {(sizes.get('rope_scaling') or {}).get('factor', 1):g}",
                   "parallelism": "single_gpu"},
        "prefill": prefill_rec,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_GBS, "unit": "GB/s", "frac": round(achieved / HBM_GBS, 4),
                     "own_peak": round(own_gbs, 1), "frac_of_own_peak": round(achieved / own_gbs, 4)},
        "points": points,
    }
    print(json.dumps(rec))
    return 0


if __name__ == "__main__":
    sys.exit(main())
