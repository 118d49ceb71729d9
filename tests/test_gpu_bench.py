"""The measurement program's own parts on a tiny model: a bench that no test runs rots."""

import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def workbench():
    sys.path.insert(0, ROOT)
    import bench
    config = {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "vocab_size": 503, "hidden_size": 192,
              "intermediate_size": 512, "num_hidden_layers": 3, "num_attention_heads": 6, "num_key_value_heads": 1,
              "head_dim": 32, "rope_theta": 1e6, "rms_norm_eps": 1e-5, "tie_word_embeddings": False,
              "max_position_embeddings": 4096}
    made = bench.Workbench(config, dtype="bfloat16", seed=0, block_size=16,
                           pool_tokens=bench.Workbench.pool_tokens([4], 256, 128), max_requests=4)
    yield bench, made
    made.close()


def test_costs_come_from_the_models_parts(workbench):
    bench, made = workbench
    h, i, v, layers, nq, nkv, d = 192, 512, 503, 3, 6, 1, 32
    matrices = layers * (h * (nq + 2 * nkv) * d + nq * d * h + 3 * h * i) + v * h          # the head; not the embedding
    vectors = layers * ((nq + 2 * nkv) * d + 2 * h) + h                                    # biases and norm weights
    assert made.weight_bytes == 2 * matrices + 4 * vectors
    assert made.cache_bytes_per_token == layers * 2 * nkv * d * 2
    tokens = 100
    pairs = tokens * (tokens + 1) // 2
    want = 2.0 * tokens * layers * (h * (nq + 2 * nkv) * d + nq * d * h + 3 * h * i) + 4.0 * nq * d * pairs * layers + 2.0 * h * v
    assert made.model.step_flops(tokens, pairs, 1) == pytest.approx(want)


def test_decode_prefill_serving_and_stage_runs(workbench):
    bench, made = workbench
    run = made.decode_run(4, 6, 2, 256)
    assert run["steps"] == 6 and len(run["step_ms"]) == 6 and 240 < run["mean_ctx"] < 320
    assert run["tok_s"] > 0 and 0 < run["frac"] < 1
    prefill = made.prefill_run(128, reps=3)
    assert prefill["tokens"] == 128 and prefill["value"] > 0 and 0 < prefill["frac"] < 1
    serving = made.serving_run(5, 4, new_tokens=8, chunk=64, budget=128, prompt_range=(8, 200))
    assert serving["requests"] == 5 and serving["generated_tokens"] == 40
    mix = serving["step_mix"]
    assert mix["live_requests"]["max"] <= 4 and mix["prompt_tokens"]["max"] <= 128 and mix["decode_tokens"]["max"] <= 4
    stages = made.stage_run(128, 2, 64)
    names = set(stages["prefill_128"])
    assert {"q/k/v", "attention", "o", "gate_up", "down", "head", "embedding", "sampling"} <= names
    assert abs(sum(r["share"] for r in stages["prefill_128"].values()) - 1.0) < 1e-2
    assert "decode_b2_eager" in stages
    assert made.runner.cache.free_pages() == [made.num_blocks] and not made.runner.cache.live_requests()


def test_bench_line_of_a_tiny_configuration_from_a_config_json(tmp_path):
    """The program end to end on a config.json of its own: one JSON line with the contract's keys, a flat config of
    at most 20 keys, points that carry their step time, context and fraction."""
    config = {"architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "vocab_size": 311, "hidden_size": 96,
              "intermediate_size": 160, "num_hidden_layers": 2, "num_attention_heads": 6, "num_key_value_heads": 2,
              "head_dim": 16, "rope_theta": 10000.0, "rms_norm_eps": 1e-6, "tie_word_embeddings": True,
              "max_position_embeddings": 2048}
    path = tmp_path / "config.json"
    path.write_text(json.dumps(config))
    out = tmp_path / "lines.jsonl"
    done = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--config-json", str(path), "--batch", "2",
                           "--context", "192", "--prefill-tokens", "64", "--steps", "4", "--warmup", "1", "--no-peaks",
                           "--no-points", "--stages", "--output-file", str(out)],
                          capture_output=True, text=True, timeout=600, cwd=str(tmp_path))
    assert done.returncode == 0, done.stderr[-2000:]
    line = json.loads(done.stdout.strip().splitlines()[-1])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "prefill", "points", "point_details", "stages"):
        assert key in line, key
    assert line["steps"] == 4 and line["n_gpus"] == 1 and line["value"] > 0
    assert len(line["config"]) <= 20 and all(not isinstance(v, (dict, list)) for v in line["config"].values())
    assert line["config"]["hidden_size"] == 96 and line["config"]["tie_word_embeddings"] is True
    assert line["roofline"]["bound"] == "hbm" and {"value", "tokens", "ms", "frac"} <= set(line["prefill"])
    assert json.loads(out.read_text().strip()) == line
    many = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                          timeout=120)
    assert many.returncode == 2 and "one GPU" in many.stdout


def test_the_machines_own_peaks_are_measured_with_the_probes():
    """The probes behind the measured peaks run: every launch shape of the streaming read over a small buffer, and the
    loop of matrix instructions on dense operands and on small integers (the same number of operations either way)."""
    import torch
    from somi_inference_amd.kernels import ops
    buffer = torch.zeros(1 << 22, dtype=torch.int32, device="cuda:0")
    shapes = ops.probe_stream_shapes()
    assert len(shapes) >= 8 and any("non-temporal" in s for s in shapes)
    for shape in shapes:
        ops.probe_stream_read(buffer, shape)
    dense = ops.probe_mfma(50, "cuda:0")
    assert dense == ops.probe_mfma(50, "cuda:0", dense=False) > 0
    torch.cuda.synchronize()
