"""bin/trace_run as a user runs it: a subprocess fed JSON lines, logits files compared with the plain
implementation for whole prompts, decoding, portions and a mixed trace with pages used again."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from helpers import TINY, assert_close, mixed_trace, token_ids
from plain import qwen2_plain as plain

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run_trace(folder, dtype, out_dir, max_tokens, steps, extra=()):
    lines = "".join(json.dumps(s) + "\n" for s in steps)
    sizing = ["--max-tokens", str(max_tokens)] if max_tokens is not None else []
    done = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
                           "--out", str(out_dir), *sizing, *extra],
                          input=lines, capture_output=True, text=True, timeout=600, cwd="/")
    assert done.returncode == 0, done.stderr[-3000:]
    assert done.stdout.split() == [w for s in steps for w in ("done", str(s["step"]))]
    return done


def read_logits(out_dir, step, vocab):
    data = np.fromfile(os.path.join(out_dir, f"{step}.f32"), dtype="<f4")
    assert data.size % vocab == 0
    return torch.from_numpy(data.reshape(-1, vocab).copy())


def round64(n):
    return (n + 63) // 64 * 64


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_replay_whole_decoded_in_portions_and_mixed(name, dtype, model_folders, tmp_path):
    folder, vocab = model_folders[name], TINY[name]["config"].vocab_size
    cfg, weights = plain.read_model(folder)
    requests = {rid: token_ids(vocab, n, 50 + i) for i, (rid, n) in enumerate({"a": 70, "b": 45, "c": 100, "d": 33, "e": 130}.items())}
    want = {rid: plain.model_logits(cfg, weights, tokens) for rid, tokens in requests.items()}

    # 1. each request alone and whole; 2. most in one step, the last 32 one by one; 3. portions down to two tokens
    steps, expect, number = [], {}, 0
    a, b, c = requests["a"], requests["b"], requests["c"]
    steps.append({"step": number, "entries": [{"id": "whole", "tokens": a, "want": list(range(len(a)))}], "end": ["whole"]})
    expect[number] = want["a"]
    number += 1
    steps.append({"step": number, "entries": [{"id": "dec", "tokens": b[:-32], "want": [len(b) - 33]}], "end": []})
    expect[number] = want["b"][len(b) - 33:len(b) - 32]
    number += 1
    for i in range(len(b) - 32, len(b)):
        steps.append({"step": number, "entries": [{"id": "dec", "tokens": [b[i]], "want": [0]}],
                      "end": ["dec"] if i == len(b) - 1 else []})
        expect[number] = want["b"][i:i + 1]
        number += 1
    at, sizes, k = 0, [7, 2, 5, 3, 11, 2, 16], 0
    while at < len(c):
        size = min(sizes[k % len(sizes)], len(c) - at)
        wanted = [0, size - 1] if size > 1 else [0]
        steps.append({"step": number, "entries": [{"id": "cut", "tokens": c[at:at + size], "want": wanted}],
                      "end": ["cut"] if at + size == len(c) else []})
        expect[number] = want["c"][[at + w for w in wanted]]
        at += size
        k += 1
        number += 1
    # the configuration's own page size: 16 for A (the program's default), 8 for B
    page = TINY[name]["block_size"]
    extra = [] if page == 16 else ["--block-size", str(page)]
    out1 = tmp_path / "single"
    run_trace(folder, dtype, out1, round64(len(c)), steps, extra)
    header = json.loads((out1 / "0.json").read_text())
    assert header["shape"] == [len(a), vocab] and header["block_size"] == page and header["dtype"] == "float32"
    assert header["rows"][3] == {"id": "whole", "place": 3, "position": 3}
    last = json.loads((out1 / f"{number - 1}.json").read_text())
    assert last["rows"][-1]["position"] == len(c) - 1
    for step, logits in expect.items():
        assert_close(read_logits(out1, step, vocab), logits, dtype, f"{name} {dtype} step {step}")
    assert not os.path.exists(out1 / "999.f32")

    # 4. mixed: up to four live requests, pool sized by the most tokens live at once (each rounded up to 64)
    trace = mixed_trace(requests, seed=9)
    live, peak = {}, 0
    for entries, ends in trace:
        for rid, start, count in entries:
            live[rid] = len(requests[rid])
        peak = max(peak, sum(round64(n) for n in live.values()))
        for rid in ends:
            del live[rid]
    assert peak < sum(round64(len(t)) for t in requests.values())
    steps, expect = [], {}
    for number, (entries, ends) in enumerate(trace):
        items, rows = [], []
        for rid, start, count in entries:
            wanted = [] if (number + start) % 5 == 0 and count > 1 else list(range(count))   # sometimes nothing is wanted
            items.append({"id": rid, "tokens": requests[rid][start:start + count], "want": wanted})
            rows.append(want[rid][[start + w for w in wanted]])
        steps.append({"step": number, "entries": items, "end": ends})
        if sum(r.shape[0] for r in rows):
            expect[number] = torch.cat(rows)
    out2 = tmp_path / "mixed"
    run_trace(folder, dtype, out2, peak, steps, extra)
    for step, logits in expect.items():
        assert_close(read_logits(out2, step, vocab), logits, dtype, f"{name} {dtype} mixed step {step}")
    assert sorted(int(f[:-4]) for f in os.listdir(out2) if f.endswith(".f32")) == sorted(expect)


def test_replay_of_seeded_random_weights_with_the_pool_given_in_pages(tmp_path):
    """--model random:<config.json>:<seed> draws the weights that the random-weights mode writes for that seed, and
    --num-blocks sizes the pool in pages: the logits equal the plain implementation's on the written folder."""
    from somi_inference_amd.weights import write_random_model
    config, seed = TINY["A"]["config"], 77
    folder = write_random_model(str(tmp_path / "written"), config, seed=seed)
    cfg, weights = plain.read_model(folder)
    tokens = token_ids(config.vocab_size, 40, 5)
    want = plain.model_logits(cfg, weights, tokens)
    steps = [{"step": 0, "entries": [{"id": "r", "tokens": tokens[:29], "want": [28]}], "end": []},
             {"step": 1, "entries": [{"id": "r", "tokens": tokens[29:], "want": list(range(11))}], "end": ["r"]}]
    out = tmp_path / "out"
    run_trace(f"random:{folder}/config.json:{seed}", "float32", out, None, steps, ["--num-blocks", "3", "--block-size", "16"])
    assert_close(read_logits(out, 0, config.vocab_size), want[28:29], "float32", "random weights, step 0")
    assert_close(read_logits(out, 1, config.vocab_size), want[29:], "float32", "random weights, step 1")
    # two pages would not hold 40 tokens
    lines = "".join(json.dumps(s) + "\n" for s in steps)
    failed = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", f"random:{folder}:{seed}",
                             "--dtype", "float32", "--out", str(tmp_path / "small"), "--num-blocks", "2"],
                            input=lines, capture_output=True, text=True, timeout=600, cwd="/")
    assert failed.returncode != 0 and "pages" in failed.stderr
