"""Decode and prefill throughput of the engine at Qwen2.5-7B layer sizes on one MI355X.

``python bench.py --gpus 1 --steps K --warmup W`` builds a random-weights model of the 7B layer
sizes in bfloat16, fills the cache of ``--batch`` requests by running their prompts through the
engine's own generation loop (scheduler, step function, sampler), then times exactly K of that loop's
decode steps (one token per request per step) between two synchronisations.  It prints ONE JSON line; ``value``
is decoded tokens per second.  The same line carries a 2,048-token prefill measurement, the decode
step's HBM roofline figures and decode throughput at batch 1 and 64.

The method follows the reference's benchmarks (warm-up, synchronise, wall clock, synchronise:
benchmarks/common.py:131-156; tokens/s = batch * iterations / time: benchmarks/bench_decode.py:241-247)
with seeded random weights and seeded uniform token ids in place of a downloaded checkpoint and a
tokenizer-built workload.  The engine runs on one GPU; for more it says so and exits with 2.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X published HBM3E bandwidth
PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}   # dense MFMA peaks
POINT_BATCHES = (1, 64, 96, 128, 256)      # decode is also measured at these numbers of requests ("points")


# layer sizes of the Qwen2.5 family: (layers, hidden, heads, kv heads, head_dim, intermediate, rms_norm_eps,
# vocabulary, tied LM head).  0.5b is the model the reference's own published figures are measured on.
LAYER_SIZES = {
    "0.5b": (24, 896, 14, 2, 64, 4864, 1e-6, 151936, True),
    "7b": (28, 3584, 28, 4, 128, 18944, 1e-6, 152064, False),
    "14b": (48, 5120, 40, 8, 128, 13824, 1e-5, 152064, False),
    "32b": (64, 5120, 40, 8, 128, 27648, 1e-6, 152064, False),
}


def parse_args() -> argparse.Namespace:
    p = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=64)
    p.add_argument("--warmup", type=int, default=8)
    p.add_argument("--batch", type=int, default=8)
    p.add_argument("--context", type=int, default=4096, help="context length the timed decode steps end at")
    p.add_argument("--sizes", default="7b", choices=sorted(LAYER_SIZES),
                   help="layer sizes: Qwen2.5-7B (the default and the headline), -14B, -32B, or -0.5B (the model of the "
                        "reference's own published figures)")
    p.add_argument("--layers", type=int, default=None, help="run fewer layers than the configuration has")
    p.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    p.add_argument("--block-size", type=int, default=16)
    p.add_argument("--prefill-tokens", type=int, default=2048)
    p.add_argument("--seed", type=int, default=0)
    p.add_argument("--no-points", action="store_true", help="skip the decode points at other batch sizes (1, 64, 96, 128, 256)")
    p.add_argument("--no-prefill", action="store_true", help="skip the prefill measurement")
    p.add_argument("--no-peaks", action="store_true", help="skip the measurement of the machine's own peaks")
    p.add_argument("--output-file", type=str, default=None, help="Append the result line to a JSONL file.")
    p.add_argument("--serving", type=int, default=0, metavar="REQUESTS",
                   help="also run this many requests (prompts of 128 to 2,048 tokens, 256 new tokens each) through "
                        "the scheduler with portions of 512, and report it under 'serving'")
    return p.parse_args()


def summarize_ms(samples_ms: list[float]) -> dict:
    """Mean, median, tail, spread and range of latency samples, as the reference summarises them
    (benchmarks/common.py:159-170)."""
    import numpy as np
    x = np.asarray(samples_ms, dtype=np.float64)
    return {"mean": round(float(x.mean()), 4), "median": round(float(np.percentile(x, 50)), 4),
            "p95": round(float(np.percentile(x, 95)), 4), "p99": round(float(np.percentile(x, 99)), 4),
            "std": round(float(x.std()), 4), "min": round(float(x.min()), 4), "max": round(float(x.max()), 4)}


def environment(device) -> dict:
    """Where the numbers come from (the reference's collect_environment_metadata, benchmarks/common.py:231-251)."""
    import platform
    import subprocess

    import torch

    def git(*args: str) -> str | None:
        try:
            done = subprocess.run(["git", *args], cwd=ROOT, capture_output=True, text=True, timeout=10)
            return done.stdout.strip() if done.returncode == 0 else None
        except (OSError, subprocess.SubprocessError):
            return None

    props = torch.cuda.get_device_properties(device)
    dirty = git("status", "--porcelain")
    return {"git_sha": git("rev-parse", "HEAD"), "git_dirty": bool(dirty) if dirty is not None else None,
            "python_version": platform.python_version(), "platform": platform.platform(),
            "torch_version": torch.__version__, "hip_version": torch.version.hip,
            "device_name": props.name, "device_arch": getattr(props, "gcnArchName", None),
            "compute_units": props.multi_processor_count, "device_memory_gb": round(props.total_memory / 2**30, 1),
            "executable": sys.executable}


def measure_peaks(device) -> dict:
    """What this machine reaches on the two resources the step is bound by: streaming memory into the compute units
    (2 GiB, beyond every cache) and bfloat16 matrix instructions on every SIMD."""
    import torch

    from somi_inference_amd.kernels import ops
    buffer = torch.empty(2 << 30, dtype=torch.uint8, device=device)
    buffer.zero_()

    def timed(fn, reps):
        fn()
        torch.cuda.synchronize()
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        for _ in range(reps):
            fn()
        end.record()
        torch.cuda.synchronize()
        return start.elapsed_time(end) / reps / 1000.0
    read_s = timed(lambda: ops.probe_stream_read(buffer), 5)
    flops = ops.probe_mfma(20000, device)
    mfma_s = timed(lambda: ops.probe_mfma(20000, device), 3)
    del buffer
    return {"stream_read_gbs": round(buffer_bytes_gb(2 << 30) / read_s, 1), "mfma_bf16_tflops": round(flops / mfma_s / 1e12, 1)}


def buffer_bytes_gb(n: int) -> float:
    return n / 1e9


def main() -> int:
    args = parse_args()
    world = int(os.environ.get("WORLD_SIZE", "1"))
    if args.gpus != 1 or world != 1:
        if int(os.environ.get("RANK", "0")) == 0:
            print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} (WORLD_SIZE {world}) is not supported")
        return 2

    import torch

    from somi_inference_amd.config import Qwen2Config
    from somi_inference_amd.engine import Engine, Request, Scheduler, StepEntry
    from somi_inference_amd.engine.engine import full_collections_deferred
    from somi_inference_amd.models import make_runner, random_model
    from somi_inference_amd.sampling import Sampler, SamplingParams

    full_layers, hidden, heads, kv_heads, head_dim, intermediate, eps, vocab, tied = LAYER_SIZES[args.sizes]
    layers = args.layers or full_layers
    config = Qwen2Config(vocab_size=vocab, hidden_size=hidden, intermediate_size=intermediate,
                         num_hidden_layers=layers, num_attention_heads=heads, num_key_value_heads=kv_heads,
                         head_dim=head_dim, rope_theta=1e6, rms_norm_eps=eps, tie_word_embeddings=tied,
                         max_position_embeddings=32768)
    torch.manual_seed(args.seed)
    device = torch.device("cuda:0")
    model = random_model(config, seed=args.seed, dtype=args.dtype, draw_on="device")
    elem = 2 if args.dtype == "bfloat16" else 4
    batches = [args.batch] if args.no_points else sorted({1, args.batch, *POINT_BATCHES})
    # Decoding is measured through the generation loop itself (scheduler, step function, sampler, running ahead of
    # the device).  The scheduler runs the prompts in portions of 2,048 tokens and lets the requests that are done
    # with theirs decode meanwhile, so a request has decoded up to `ramp` tokens before the timed steps begin.
    portion = 2048
    # (beyond 128 requests the decoding tokens take a visible share of a step's 2,048: a prompt then needs one portion more)
    ramp = max(batches) * ((args.context + portion - 1) // portion + (1 if max(batches) > 128 else 0)) + 8
    pages_per_request = (args.context + ramp + args.block_size - 1) // args.block_size + 1
    num_blocks = max(max(batches) * pages_per_request,
                     (args.prefill_tokens + args.block_size - 1) // args.block_size + 1)
    runner = make_runner(model, block_size=args.block_size, num_blocks=num_blocks, max_requests=max(batches) + 1)
    sampler, greedy = Sampler(), SamplingParams(temperature=0.0)
    gen = torch.Generator().manual_seed(args.seed)

    weight_bytes = sum(t.numel() * t.element_size() for t in _decode_weights(model))
    kv_bytes_per_token = 2 * config.num_key_value_heads * config.head_dim * elem * layers

    def sync() -> None:
        torch.cuda.synchronize()

    def decode_run(batch: int, steps: int, warmup: int) -> dict:
        """``batch`` requests whose prompts end ``warmup + steps`` tokens before the context length, run by the
        engine; times ``steps`` of its decode steps.  Every step is one scheduling decision, one model step for all
        requests and one sampling call, launched ahead of the device as generation does it."""
        scheduler = Scheduler(runner.cache, max_concurrent=batch, max_num_batched_tokens=max(portion, batch), chunk=portion)
        engine = Engine(runner, scheduler, sampler, eos_token_id=-1)
        prompt_len = args.context - (warmup + steps + 1)
        requests = [Request(f"b{batch}_{i}", torch.randint(0, config.vocab_size, (prompt_len,), generator=gen).tolist(),
                            ramp + warmup + steps + 8, greedy, seed=i) for i in range(batch)]
        runner.capture_decode_graphs(batch, args.context + ramp)
        for request in requests:
            engine.add_request(request)
        with full_collections_deferred():          # as Engine.run() steps its requests
            while scheduler.waiting or any(r.num_computed < len(r.prompt_tokens) for r in requests):
                engine.step()
            for _ in range(warmup):
                engine.step()
            sync()
            cached_before = sum(runner.cache.num_tokens(r.request_id) for r in requests)
            marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
            marks[0].record()
            start = time.perf_counter()
            for i in range(steps):
                engine.step()
                marks[i + 1].record()
            sync()
            seconds = time.perf_counter() - start
        cached_after = sum(runner.cache.num_tokens(r.request_id) for r in requests)
        assert cached_after - cached_before == batch * steps, "a timed step was not a decode step of every request"
        step_ms = [marks[i].elapsed_time(marks[i + 1]) for i in range(steps)]
        engine.abort(requests)
        return dict(tok_s=batch * steps / seconds, ms=1000.0 * seconds / steps, steps=steps, warmup=warmup,
                    mean_ctx=(cached_before + cached_after) / 2.0 / batch, step_ms=step_ms,
                    run_ahead=engine.steps_run_ahead)

    results = {}
    for batch in batches:
        steps = args.steps if batch == args.batch else max(8, args.steps // (2 if batch <= 64 else 4))
        warmup = args.warmup if batch == args.batch else max(2, args.warmup // 2)
        results[batch] = decode_run(batch, steps, warmup)

    main_run = results[args.batch]
    step_bytes = weight_bytes + args.batch * main_run["mean_ctx"] * kv_bytes_per_token
    achieved = step_bytes / (main_run["ms"] / 1000.0) / 1e9
    peaks = None if args.no_peaks else measure_peaks(device)

    prefill = None
    if not args.no_prefill:
        tokens = torch.randint(0, config.vocab_size, (args.prefill_tokens,), generator=gen).tolist()
        times = []
        for rep in range(6):
            runner.begin("prefill")
            sync()
            start = time.perf_counter()
            runner.step([StepEntry("prefill", tokens, [len(tokens) - 1])])
            sync()
            times.append(time.perf_counter() - start)
            runner.end("prefill")
        times = sorted(times[1:])                     # the first run pays one-time set-up
        seconds = times[len(times) // 2]              # the median of five
        flops = _prefill_flops(config, args.prefill_tokens)
        prefill = {"value": round(args.prefill_tokens / seconds, 1), "tokens": args.prefill_tokens,
                   "ms": round(seconds * 1000.0, 3), "frac": round(flops / seconds / PEAK_FLOPS[args.dtype], 4),
                   "ms_min": round(times[0] * 1000.0, 3), "ms_max": round(times[-1] * 1000.0, 3)}
        if peaks is not None and args.dtype == "bfloat16":
            prefill["frac_of_measured_mfma"] = round(flops / seconds / (peaks["mfma_bf16_tflops"] * 1e12), 4)

    serving = None
    if args.serving > 0:
        # continuous batching through the engine's own scheduler: everything arrives at once, prompts are cut
        # into portions of 512 under a budget of 2,048 tokens a step, finished requests free their pages
        from collections import deque
        lengths = torch.randint(128, 2049, (args.serving,), generator=gen).tolist()
        new_tokens = 256
        # the pool made for the decode runs serves here too; at most as many requests at once as fit whole
        per_request = (2048 + new_tokens + args.block_size - 1) // args.block_size + 1
        concurrent = max(1, min(args.serving, max(batches), num_blocks // per_request))
        scheduler = Scheduler(runner.cache, max_concurrent=concurrent, max_num_batched_tokens=2048, chunk=512)
        engine = Engine(runner, scheduler, sampler, eos_token_id=-1)
        arrivals = deque((0, Request(f"s{i}", torch.randint(0, config.vocab_size, (n,), generator=gen).tolist(),
                                     new_tokens, greedy, seed=i)) for i, n in enumerate(lengths))
        # as LLM.warm_up() does it: the decode graphs that the requests will replay are captured before they arrive
        captured = runner.capture_decode_graphs(concurrent, 2048 + new_tokens)
        sync()
        start = time.perf_counter()
        done = engine.run(arrivals)
        sync()
        seconds = time.perf_counter() - start
        generated = sum(len(r.output_tokens) for r in done)
        serving = {"requests": len(done), "prompt_tokens": sum(lengths), "generated_tokens": generated,
                   "seconds": round(seconds, 3), "generated_tok_s": round(generated / seconds, 1),
                   "total_tok_s": round((generated + sum(lengths)) / seconds, 1), "steps": engine.num_steps,
                   "steps_run_ahead": engine.steps_run_ahead, "max_concurrent": concurrent,
                   "preemptions": sum(r.num_preemptions for r in done), "graphs_captured_ahead": captured}

    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4)}
    if peaks is not None:
        roofline["measured_peak"] = peaks["stream_read_gbs"]
        roofline["frac_of_measured"] = round(achieved / peaks["stream_read_gbs"], 4)
    line = {
        "metric": f"decode tok/s at batch {args.batch}, Qwen2.5-{args.sizes.upper()} layer sizes "
                  f"(plus prefill tok/s at {args.prefill_tokens:,} tokens, batch 1/64/96/128/256 points)",
        "value": round(main_run["tok_s"], 2), "unit": "tokens/s", "n_gpus": 1,
        "steps": main_run["steps"], "warmup": main_run["warmup"], "ms_per_step": round(main_run["ms"], 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: seeded random N(0,0.02) weights, seeded uniform token ids; prompts run and tokens decoded "
                "by the engine's own generation loop",
        "config": {"model": f"Qwen2.5-{args.sizes.upper()} layer sizes (random weights)", "global_batch": args.batch,
                   "seq_len": args.context, "parallelism": "single GPU", "layers": layers,
                   "layers_of_config": full_layers, "hidden_size": config.hidden_size,
                   "intermediate_size": config.intermediate_size, "num_attention_heads": config.num_attention_heads,
                   "num_key_value_heads": config.num_key_value_heads, "head_dim": config.head_dim,
                   "vocab_size": config.vocab_size, "tie_word_embeddings": tied, "block_size": args.block_size,
                   "mean_context": round(main_run["mean_ctx"], 1)},
        "roofline": roofline,
        "latency_ms": summarize_ms(main_run["step_ms"]),
        "points": {f"decode_b{b}": round(r["tok_s"], 2) for b, r in results.items() if b in POINT_BATCHES},
    }
    if prefill is not None:
        line["prefill"] = prefill
    if serving is not None:
        line["serving"] = serving
    if peaks is not None:
        line["measured_peaks"] = peaks
    line["environment"] = environment(device)
    text = json.dumps(line)
    print(text)
    if args.output_file:
        os.makedirs(os.path.dirname(os.path.abspath(args.output_file)), exist_ok=True)
        with open(args.output_file, "a", encoding="utf-8") as handle:      # appended, as the reference's runs are
            handle.write(text + "\n")
    return 0


def _decode_weights(model):
    """Every weight a decode step reads once: all layers' matrices, norms, biases and the head
    (the embedding table is touched for one row per request only)."""
    seen, out = set(), []
    for layer in model.layers:
        for part in layer.parts():
            for value in vars(part).values():
                tensors = []
                if hasattr(value, "weight") and hasattr(value, "bias"):
                    tensors = [value.weight, value.bias]
                elif hasattr(value, "data_ptr"):
                    tensors = [value]
                for t in tensors:
                    if t is not None and t.data_ptr() not in seen:
                        seen.add(t.data_ptr())
                        out.append(t)
    for t in (model.final_norm.weight, model.head.weight):
        if t.data_ptr() not in seen:
            seen.add(t.data_ptr())
            out.append(t)
    return out


def _prefill_flops(config, tokens: int) -> float:
    h, i, d = config.hidden_size, config.intermediate_size, config.head_dim
    nq, nkv, layers = config.num_attention_heads, config.num_key_value_heads, config.num_hidden_layers
    linear = 2.0 * tokens * (h * (nq + 2 * nkv) * d + nq * d * h + 3 * h * i) * layers
    attention = 4.0 * nq * d * (tokens * (tokens + 1) / 2.0) * layers     # q.k and p.v over the causal half
    head = 2.0 * h * config.vocab_size                                    # logits of the last position only
    return linear + attention + head


if __name__ == "__main__":
    sys.exit(main())
