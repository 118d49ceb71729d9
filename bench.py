"""Decode and prefill throughput of the engine on one MI355X, at the layer sizes of Qwen2.5-7B by default.

``python bench.py --gpus 1 --steps K --warmup W`` builds a random-weights model in bfloat16, fills the cache of
``--batch`` requests by running their prompts through the engine's own generation loop (scheduler, step function,
sampler), then times exactly K of that loop's decode steps (one token per request per step) between two
synchronisations.  It prints ONE JSON line; ``value`` is decoded tokens per second.  The same line carries a
2,048-token prefill measurement, the decode step's HBM roofline figures, decode throughput at other numbers of
requests (``points``, with their step times, contexts and roofline fractions under ``point_details``) and, in the
default run, shorter measurements at the other configurations the headline is quoted beside (``extras``: the
14B sizes decoding and serving 32 requests with prompts in portions, the 32B sizes at 8,192 tokens, the 7B sizes at
32,768 tokens), each reported as an error instead of failing the line.

The model is whatever the registry builds from a config.json (``--config-json``, default: the ``--sizes`` of the
Qwen2.5 family): the bytes a decode step must read come from the tensors the model's parts declare and from its
cache specs, the operations of a prefill from the parts' own counts.  ``--stages`` adds the share of each named
stage (embedding, each product, attention, sampling) in eager steps.

The method follows the reference's benchmarks (warm-up, synchronise, wall clock, synchronise:
benchmarks/common.py:131-156; tokens/s = batch * iterations / time: benchmarks/bench_decode.py:241-247; the
engine run as a whole with its arrivals: benchmarks/bench_engine.py:181-283) with seeded random weights and seeded
uniform token ids in place of a downloaded checkpoint and a tokenizer-built workload.  The engine runs on one GPU;
for more it says so and exits with 2.
"""

from __future__ import annotations

import argparse
import gc
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X published HBM3E bandwidth
PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}   # dense MFMA peaks
POINT_BATCHES = (1, 64, 96, 128, 256)      # decode is also measured at these numbers of requests ("points")
POINT_MIN_STEPS = 16                       # a point is timed over at least this many steps


# layer sizes of the Qwen2.5 family: (layers, hidden, heads, kv heads, head_dim, intermediate, rms_norm_eps,
# vocabulary, tied LM head).  0.5b is the model the reference's own published figures are measured on.
LAYER_SIZES = {
    "0.5b": (24, 896, 14, 2, 64, 4864, 1e-6, 151936, True),
    "7b": (28, 3584, 28, 4, 128, 18944, 1e-6, 152064, False),
    "14b": (48, 5120, 40, 8, 128, 13824, 1e-5, 152064, False),
    "32b": (64, 5120, 40, 8, 128, 27648, 1e-6, 152064, False),
}
# keys of a config.json that name sizes, in the order they are reported under "config" (flat, at most 20 keys)
SIZE_KEYS = ("hidden_size", "intermediate_size", "num_attention_heads", "num_key_value_heads", "head_dim",
             "vocab_size", "tie_word_embeddings")


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
    p.add_argument("--config-json", type=str, default=None,
                   help="a config.json of any registered architecture instead of --sizes")
    p.add_argument("--layers", type=int, default=None, help="run fewer layers than the configuration has")
    p.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    p.add_argument("--block-size", type=int, default=16)
    p.add_argument("--prefill-tokens", type=int, default=2048)
    p.add_argument("--seed", type=int, default=0)
    p.add_argument("--no-points", action="store_true", help="skip the decode points at other batch sizes (1, 64, 96, 128, 256)")
    p.add_argument("--no-prefill", action="store_true", help="skip the prefill measurement")
    p.add_argument("--no-peaks", action="store_true", help="skip the measurement of the machine's own peaks")
    p.add_argument("--no-extras", action="store_true",
                   help="skip the short measurements at the 14B and 32B sizes and at 32,768 tokens that the default run adds")
    p.add_argument("--extras-budget", type=float, default=300.0, metavar="SECONDS",
                   help="no further extra measurement is started once the run has taken this long")
    p.add_argument("--stages", action="store_true",
                   help="also time the named stages of an eager prefill and an eager decode step and report their shares")
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


def summarize_counts(samples: list[int]) -> dict:
    import numpy as np
    x = np.asarray(samples or [0], dtype=np.float64)
    return {"mean": round(float(x.mean()), 1), "median": float(np.percentile(x, 50)), "max": float(x.max())}


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
    (2 GiB, beyond every cache; the best of the read kernel's launch shapes) and bfloat16 matrix instructions on
    every SIMD."""
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
    shapes = {}
    for shape in ops.probe_stream_shapes():
        shapes[shape] = round((2 << 30) / 1e9 / timed(lambda: ops.probe_stream_read(buffer, shape), 5), 1)
    # matrix instructions on operands as a product has them, and on small integers (most bits zero: the clock under
    # matrix instructions goes with what the operands toggle, so this loop runs faster than any product can)
    flops = ops.probe_mfma(20000, device)
    mfma_s = timed(lambda: ops.probe_mfma(20000, device), 3)
    sparse_s = timed(lambda: ops.probe_mfma(20000, device, dense=False), 3)
    del buffer
    best = max(shapes, key=shapes.get)
    return {"stream_read_gbs": shapes[best], "stream_read_shape": best, "stream_read_by_shape": shapes,
            "mfma_bf16_tflops": round(flops / mfma_s / 1e12, 1),
            "mfma_bf16_tflops_small_integers": round(flops / sparse_s / 1e12, 1)}


def qwen2_config_dict(sizes: str, layers: int | None) -> dict:
    """The config.json of the Qwen2.5 layer sizes named ``sizes`` (with fewer layers if asked)."""
    full_layers, hidden, heads, kv_heads, head_dim, intermediate, eps, vocab, tied = LAYER_SIZES[sizes]
    return {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "vocab_size": vocab, "hidden_size": hidden,
            "intermediate_size": intermediate, "num_hidden_layers": layers or full_layers,
            "num_attention_heads": heads, "num_key_value_heads": kv_heads, "head_dim": head_dim, "rope_theta": 1e6,
            "rms_norm_eps": eps, "tie_word_embeddings": tied, "max_position_embeddings": 32768,
            "hidden_act": "silu", "attention_bias": True}


class Workbench:
    """One model on the GPU with a cache pool, and the measurements that run on it.  The model comes from the
    registry by the architecture its config.json names; what a step costs is asked of the model's parts."""

    def __init__(self, config_dict: dict, *, dtype: str, seed: int, block_size: int, pool_tokens: int,
                 max_requests: int) -> None:
        import torch

        from somi_inference_amd.cache import CacheManager
        from somi_inference_amd.config.registry import config_from_dict
        from somi_inference_amd.models import make_runner, random_model
        from somi_inference_amd.sampling import Sampler, SamplingParams

        self.torch = torch
        _, self.config = config_from_dict(config_dict)
        self.config_dict = config_dict
        self.dtype, self.block_size = dtype, block_size
        self.device = torch.device("cuda:0")
        self.model = random_model(self.config, seed=seed, dtype=dtype, draw_on="device")
        self.num_blocks = (pool_tokens + block_size - 1) // block_size + max_requests + 1
        self.runner = make_runner(self.model, block_size=block_size, num_blocks=self.num_blocks, max_requests=max_requests + 1)
        self.sampler, self.greedy = Sampler(), SamplingParams(temperature=0.0)
        self.gen = torch.Generator().manual_seed(seed)
        self.vocab = self.model.vocab_size
        self.weight_bytes = self.model.step_weight_bytes()
        self.cache_bytes_per_token = CacheManager.page_bytes(self.model.cache_needs(), block_size,
                                                             self.model.runtime.dtype) / block_size

    def close(self) -> None:
        """Give the device memory back (weights, pool, captured graphs) before another model is built."""
        self.runner._graphs.clear()
        self.runner = self.model = self.sampler = None
        gc.collect()
        self.torch.cuda.empty_cache()

    def tokens(self, count: int) -> list[int]:
        return self.torch.randint(0, self.vocab, (count,), generator=self.gen).tolist()

    def decode_bytes(self, batch: int, mean_context: float) -> float:
        """What a decode step has to read: every weight once and the cache of the live requests."""
        return self.weight_bytes + batch * mean_context * self.cache_bytes_per_token

    # ------------------------------------------------------------------ decode
    def decode_run(self, batch: int, steps: int, warmup: int, context: int, portion: int = 2048) -> dict:
        """``batch`` requests whose prompts end ``warmup + steps`` tokens before the context length, run by the
        engine; times ``steps`` of its decode steps.  Every step is one scheduling decision, one model step for all
        requests and one sampling call, launched ahead of the device as generation does it.  The scheduler runs the
        prompts in portions and lets the requests that are done with theirs decode meanwhile, so a request has
        decoded some tokens before the timed steps begin (``mean_ctx`` says where the timed steps stood)."""
        from somi_inference_amd.engine import Engine, Request, Scheduler
        from somi_inference_amd.engine.engine import full_collections_deferred
        torch, runner = self.torch, self.runner
        scheduler = Scheduler(runner.cache, max_concurrent=batch, max_num_batched_tokens=max(portion, batch), chunk=portion)
        engine = Engine(runner, scheduler, self.sampler, eos_token_id=-1)
        prompt_len = context - (warmup + steps + 1)
        ramp = self.ramp(batch, context, portion)
        requests = [Request(f"b{batch}_{i}", self.tokens(prompt_len), ramp + warmup + steps + 8, self.greedy, seed=i)
                    for i in range(batch)]
        runner.capture_decode_graphs(batch, context + ramp)
        for request in requests:
            engine.add_request(request)
        with full_collections_deferred():          # as Engine.run() steps its requests
            while scheduler.waiting or any(r.num_computed < len(r.prompt_tokens) for r in requests):
                engine.step()
            for _ in range(warmup):
                engine.step()
            torch.cuda.synchronize()
            cached_before = sum(runner.cache.num_tokens(r.request_id) for r in requests)
            marks = [torch.cuda.Event(enable_timing=True) for _ in range(steps + 1)]
            marks[0].record()
            start = time.perf_counter()
            for i in range(steps):
                engine.step()
                marks[i + 1].record()
            torch.cuda.synchronize()
            seconds = time.perf_counter() - start
        cached_after = sum(runner.cache.num_tokens(r.request_id) for r in requests)
        assert cached_after - cached_before == batch * steps, "a timed step was not a decode step of every request"
        step_ms = [marks[i].elapsed_time(marks[i + 1]) for i in range(steps)]
        engine.abort(requests)
        mean_ctx = (cached_before + cached_after) / 2.0 / batch
        ms = 1000.0 * seconds / steps
        achieved = self.decode_bytes(batch, mean_ctx) / (ms / 1000.0) / 1e9
        return dict(tok_s=batch * steps / seconds, ms=ms, steps=steps, warmup=warmup, mean_ctx=mean_ctx,
                    step_ms=step_ms, run_ahead=engine.steps_run_ahead, achieved_gbs=achieved,
                    frac=achieved / HBM_PEAK_GBS)

    @staticmethod
    def ramp(batch: int, context: int, portion: int = 2048) -> int:
        """Tokens a request may decode while the others' prompts are still run, at most (beyond 128 requests the
        decoding tokens take a visible share of a step's tokens: a prompt then needs one portion more)."""
        return batch * ((context + portion - 1) // portion + (1 if batch > 128 else 0)) + 8

    @classmethod
    def pool_tokens(cls, batches, context: int, prefill_tokens: int = 0) -> int:
        most = max(batches)
        return max(most * (context + cls.ramp(most, context) + 32), prefill_tokens + 32)

    # ----------------------------------------------------------------- prefill
    def prefill_run(self, tokens: int, reps: int = 6) -> dict:
        from somi_inference_amd.engine import StepEntry
        torch, runner = self.torch, self.runner
        prompt = self.tokens(tokens)
        times = []
        for _ in range(reps):
            runner.begin("prefill")
            torch.cuda.synchronize()
            start = time.perf_counter()
            runner.step([StepEntry("prefill", prompt, [len(prompt) - 1])])
            torch.cuda.synchronize()
            times.append(time.perf_counter() - start)
            runner.end("prefill")
        times = sorted(times[1:])                     # the first run pays one-time set-up
        seconds = times[len(times) // 2]              # the median of the others
        flops = self.model.step_flops(tokens, tokens * (tokens + 1) // 2, 1)
        return {"value": round(tokens / seconds, 1), "tokens": tokens, "ms": round(seconds * 1000.0, 3),
                "frac": round(flops / seconds / PEAK_FLOPS[self.dtype], 4), "ms_min": round(times[0] * 1000.0, 3),
                "ms_max": round(times[-1] * 1000.0, 3), "tflop": round(flops / 1e12, 3)}

    # ----------------------------------------------------------------- serving
    def serving_run(self, count: int, max_concurrent: int, new_tokens: int = 256, chunk: int = 512,
                    budget: int = 2048, prompt_range: tuple[int, int] = (128, 2048)) -> dict:
        """Continuous batching through the engine's own scheduler: everything arrives at once, prompts of
        ``prompt_range`` tokens (128 to 2,048) are cut into portions of ``chunk`` under a budget of ``budget`` tokens a step, finished requests
        free their pages.  Reported as a whole, with what a step held (the reference reports a run with its arrival
        trace: benchmarks/bench_engine.py:181-283)."""
        from somi_inference_amd.engine import Engine, Request, Scheduler
        from somi_inference_amd.engine.engine import full_collections_deferred
        torch, runner = self.torch, self.runner
        shortest, longest = prompt_range
        lengths = torch.randint(shortest, longest + 1, (count,), generator=self.gen).tolist()
        per_request = (longest + new_tokens + self.block_size - 1) // self.block_size + 1
        concurrent = max(1, min(count, max_concurrent, self.num_blocks // per_request))
        scheduler = Scheduler(runner.cache, max_concurrent=concurrent, max_num_batched_tokens=budget, chunk=chunk)
        engine = Engine(runner, scheduler, self.sampler, eos_token_id=-1)
        requests = [Request(f"s{i}", self.tokens(n), new_tokens, self.greedy, seed=i) for i, n in enumerate(lengths)]
        # as LLM.warm_up() does it: the decode graphs that the requests will replay are captured before they arrive
        captured = runner.capture_decode_graphs(concurrent, longest + new_tokens)
        prompt_mix, decode_mix, live_mix = [], [], []
        torch.cuda.synchronize()
        start = time.perf_counter()
        for request in requests:
            engine.add_request(request)
        done = []
        with full_collections_deferred():
            while scheduler.has_unfinished():
                done.extend(engine.step())
                portions = engine.last_output.portions
                decoding = sum(1 for p in portions if p.start >= len(p.request.prompt_tokens))
                decode_mix.append(decoding)
                prompt_mix.append(sum(len(p.tokens) for p in portions) - decoding)
                live_mix.append(len(portions))
        done.extend(engine.run())                     # reads the last step's tokens
        torch.cuda.synchronize()
        seconds = time.perf_counter() - start
        generated = sum(len(r.output_tokens) for r in requests)
        assert all(len(r.output_tokens) == new_tokens for r in requests), "a request did not finish"
        return {"requests": len(requests), "prompt_tokens": sum(lengths), "generated_tokens": generated,
                "seconds": round(seconds, 3), "generated_tok_s": round(generated / seconds, 1),
                "total_tok_s": round((generated + sum(lengths)) / seconds, 1), "steps": engine.num_steps,
                "steps_run_ahead": engine.steps_run_ahead, "max_concurrent": concurrent,
                "preemptions": sum(r.num_preemptions for r in requests), "graphs_captured_ahead": captured,
                "step_mix": {"prompt_tokens": summarize_counts(prompt_mix), "decode_tokens": summarize_counts(decode_mix),
                             "live_requests": summarize_counts(live_mix)}}

    # ------------------------------------------------------------------ stages
    def stage_run(self, prefill_tokens: int, batch: int, context: int) -> dict:
        """Shares of the named stages in an eager prefill and in an eager decode step of ``batch`` requests at
        ``context`` tokens (captured graphs hold no stages, so the decode step is run without them)."""
        from somi_inference_amd.engine import StepEntry
        from somi_inference_amd.kernels import stages
        torch, runner = self.torch, self.runner
        out = {}
        prompt = self.tokens(prefill_tokens)
        for rep in range(2):                          # the second run is the one that counts
            runner.begin("stages")
            with stages.collect() as times:
                logits = runner.step([StepEntry("stages", prompt, [len(prompt) - 1])])
                self.sampler.sample(logits, self.greedy)
            out[f"prefill_{prefill_tokens}"] = times.summary()
            runner.end("stages")
        ids = [f"stage{i}" for i in range(batch)]
        for rid in ids:
            runner.begin(rid)
            runner.step([StepEntry(rid, self.tokens(context - 3), [])])
        graphs, runner.decode_graphs = runner.decode_graphs, False
        try:
            for rep in range(2):
                with stages.collect() as times:
                    logits = runner.step([StepEntry(rid, [1], [0]) for rid in ids])
                    self.sampler.sample(logits, [self.greedy] * batch)
                out[f"decode_b{batch}_eager"] = times.summary()
        finally:
            runner.decode_graphs = graphs
            for rid in ids:
                runner.end(rid)
        torch.cuda.synchronize()
        return out


def print_stage_tables(stage_times: dict) -> None:
    for what, rows in stage_times.items():
        total = sum(r["ms"] for r in rows.values())
        print(f"\n{what}: {total:.3f} ms in named stages", file=sys.stderr)
        print(f"  {'stage':<36}{'calls':>7}{'ms':>11}{'share':>9}", file=sys.stderr)
        for name, r in rows.items():
            print(f"  {name:<36}{r['calls']:>7}{r['ms']:>11.3f}{100 * r['share']:>8.1f}%", file=sys.stderr)


def config_block(bench: Workbench, label: str, batch: int, context: int, layers_of_config: int, mean_ctx: float) -> dict:
    data = bench.config.to_dict() if hasattr(bench.config, "to_dict") else dict(bench.config_dict)
    block = {"model": label, "global_batch": batch, "seq_len": context, "parallelism": "single GPU",
             "layers": data.get("num_hidden_layers"), "layers_of_config": layers_of_config}
    for key in SIZE_KEYS:
        if key in data and isinstance(data[key], (int, float, bool, str)):
            block[key] = data[key]
    block["block_size"] = bench.block_size
    block["mean_context"] = round(mean_ctx, 1)
    return block


def run_extras(args, started: float) -> dict:
    """Short measurements at the other configurations: each in a block of its own that reports an error instead of
    failing the line, none started once the run has taken ``--extras-budget`` seconds."""
    extras: dict = {}

    def within_budget(name: str) -> bool:
        if time.perf_counter() - started > args.extras_budget:
            extras[name] = {"skipped": f"the run had taken more than {args.extras_budget:.0f} s"}
            return False
        return True

    def point(run: dict) -> dict:
        return {"tok_s": round(run["tok_s"], 1), "ms": round(run["ms"], 4), "mean_ctx": round(run["mean_ctx"], 1),
                "frac": round(run["frac"], 4), "steps": run["steps"]}

    def attempt(name: str, fn) -> None:
        if not within_budget(name):
            return
        bench = None
        try:
            t0 = time.perf_counter()
            bench, result = fn()
            result["seconds_taken"] = round(time.perf_counter() - t0, 1)
            extras[name] = result
        except Exception as err:      # noqa: BLE001 - an extra must not fail the line
            extras[name] = {"error": f"{type(err).__name__}: {err}"[:300]}
        finally:
            import torch
            if bench is not None:
                bench.close()
            gc.collect()
            torch.cuda.empty_cache()

    def long_context():
        context = 32768
        bench = Workbench(qwen2_config_dict("7b", None), dtype=args.dtype, seed=args.seed, block_size=args.block_size,
                          pool_tokens=Workbench.pool_tokens([8], context), max_requests=8)
        return bench, {"sizes": "7b", "decode_b8": point(bench.decode_run(8, 16, 2, context))}

    def sizes_14b():
        bench = Workbench(qwen2_config_dict("14b", None), dtype=args.dtype, seed=args.seed, block_size=args.block_size,
                          pool_tokens=Workbench.pool_tokens([64], 4096), max_requests=64)
        result = {"sizes": "14b", "layers": 48}
        for batch in (8, 64):
            result[f"decode_b{batch}"] = point(bench.decode_run(batch, 16, 2, 4096))
        result["serving_32_requests"] = bench.serving_run(32, 32)
        return bench, result

    def sizes_32b():
        context = 8192
        bench = Workbench(qwen2_config_dict("32b", None), dtype=args.dtype, seed=args.seed, block_size=args.block_size,
                          pool_tokens=Workbench.pool_tokens([64], context), max_requests=64)
        result = {"sizes": "32b", "layers": 64, "prefill": bench.prefill_run(context, reps=3)}
        result["decode_b64"] = point(bench.decode_run(64, 16, 2, context))
        return bench, result

    attempt("long_context_7b", long_context)
    attempt("qwen2.5_14b", sizes_14b)
    attempt("qwen2.5_32b", sizes_32b)
    return extras


def main() -> int:
    args = parse_args()
    world = int(os.environ.get("WORLD_SIZE", "1"))
    if args.gpus != 1 or world != 1:
        if int(os.environ.get("RANK", "0")) == 0:
            print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} (WORLD_SIZE {world}) is not supported")
        return 2
    started = time.perf_counter()

    import torch

    if args.config_json:
        with open(args.config_json, "r", encoding="utf-8") as handle:
            config_dict = json.load(handle)
        layers_of_config = int(config_dict.get("num_hidden_layers", 0))
        if args.layers:
            config_dict["num_hidden_layers"] = args.layers
        label = f"{(config_dict.get('architectures') or ['?'])[0]} from {os.path.basename(os.path.abspath(args.config_json))} (random weights)"
        name = label
    else:
        layers_of_config = LAYER_SIZES[args.sizes][0]
        config_dict = qwen2_config_dict(args.sizes, args.layers)
        label = f"Qwen2.5-{args.sizes.upper()} layer sizes (random weights)"
        name = f"Qwen2.5-{args.sizes.upper()} layer sizes"
    torch.manual_seed(args.seed)
    batches = [args.batch] if args.no_points else sorted({1, args.batch, *POINT_BATCHES})
    bench = Workbench(config_dict, dtype=args.dtype, seed=args.seed, block_size=args.block_size,
                      pool_tokens=Workbench.pool_tokens(batches, args.context, args.prefill_tokens),
                      max_requests=max(batches))

    results = {}
    for batch in batches:
        steps = args.steps if batch == args.batch else max(POINT_MIN_STEPS, args.steps // (2 if batch <= 64 else 4))
        warmup = args.warmup if batch == args.batch else max(2, args.warmup // 2)
        results[batch] = bench.decode_run(batch, steps, warmup, args.context)
    main_run = results[args.batch]
    peaks = None if args.no_peaks else measure_peaks(bench.device)

    prefill = None
    if not args.no_prefill:
        prefill = bench.prefill_run(args.prefill_tokens)
        if peaks is not None and args.dtype == "bfloat16":
            prefill["frac_of_measured_mfma"] = round(prefill["tflop"] * 1e12 / (prefill["ms"] / 1000.0)
                                                     / (peaks["mfma_bf16_tflops"] * 1e12), 4)
    serving = bench.serving_run(args.serving, max(batches)) if args.serving > 0 else None
    stage_times = bench.stage_run(args.prefill_tokens, args.batch, args.context) if args.stages else None

    roofline = {"bound": "hbm", "achieved": round(main_run["achieved_gbs"], 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(main_run["frac"], 4)}
    if peaks is not None:
        roofline["measured_peak"] = peaks["stream_read_gbs"]
        roofline["frac_of_measured"] = round(main_run["achieved_gbs"] / peaks["stream_read_gbs"], 4)
    line = {
        "metric": f"decode tok/s at batch {args.batch}, {name} "
                  f"(plus prefill tok/s at {args.prefill_tokens:,} tokens, batch 1/64/96/128/256 points)",
        "value": round(main_run["tok_s"], 2), "unit": "tokens/s", "n_gpus": 1,
        "steps": main_run["steps"], "warmup": main_run["warmup"], "ms_per_step": round(main_run["ms"], 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic: seeded random N(0,0.02) weights, seeded uniform token ids; prompts run and tokens decoded "
                "by the engine's own generation loop",
        "config": config_block(bench, label, args.batch, args.context, layers_of_config, main_run["mean_ctx"]),
        "roofline": roofline,
        "latency_ms": summarize_ms(main_run["step_ms"]),
        "points": {f"decode_b{b}": round(r["tok_s"], 2) for b, r in results.items() if b in POINT_BATCHES},
        "point_details": {f"decode_b{b}": {"ms": round(r["ms"], 4), "mean_ctx": round(r["mean_ctx"], 1),
                                           "frac": round(r["frac"], 4), "steps": r["steps"]}
                          for b, r in results.items() if b in POINT_BATCHES},
    }
    if prefill is not None:
        line["prefill"] = prefill
    if serving is not None:
        line["serving"] = serving
    if peaks is not None:
        line["measured_peaks"] = peaks
    if stage_times is not None:
        line["stages"] = stage_times
        print_stage_tables(stage_times)
    line["environment"] = environment(bench.device)
    default_run = not args.config_json and args.sizes == "7b" and not args.layers and not args.no_points
    if default_run and not args.no_extras:
        bench.close()
        line["extras"] = run_extras(args, started)
    line["seconds_total"] = round(time.perf_counter() - started, 1)
    text = json.dumps(line)
    print(text)
    if args.output_file:
        os.makedirs(os.path.dirname(os.path.abspath(args.output_file)), exist_ok=True)
        with open(args.output_file, "a", encoding="utf-8") as handle:      # appended, as the reference's runs are
            handle.write(text + "\n")
    return 0


if __name__ == "__main__":
    sys.exit(main())
