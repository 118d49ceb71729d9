"""Trace replay: feeds given token ids through the model step by step and writes logits.

It samples nothing and owns no forward pass, cache or loader: it drives the
model, step function and cache manager that generation uses.  The nearest thing
in the reference is the hand-written prefill/decode loop of
tests/models/test_qwen2_e2e.py:65-77.

Input, one JSON object per line::

    {"step": 0, "entries": [{"id": "a", "tokens": [5, 17, 3], "want": [0, 2]}], "end": []}

For a step with wanted places the logits are written to ``<out>/<step>.f32`` as
little-endian float32 ``[wanted, vocab]``, in the order of the entries and of
``want``.  After every step a line ``done <step>`` is printed and flushed.
"""

from __future__ import annotations

import json
import os
import sys
from typing import IO

import numpy as np

from ..config.base import read_config_json
from ..config.registry import config_from_dict
from ..engine.batch import StepEntry
from ..models.loader import load_model, make_runner, random_model

DEFAULT_PAGE_TOKENS = 16      # tokens per cache page unless asked otherwise; divides the 64 that --max-tokens is counted in
DEFAULT_MAX_REQUESTS = 64     # request slots of the cache manager (a trace holds a handful live)
RANDOM_PREFIX = "random:"


def open_model(model: str, dtype: str, device: str):
    """``model``: a folder with config.json and model.safetensors, or ``random:<config.json>:<seed>`` for seeded
    random weights of the configuration in that file (a folder with a config.json works too)."""
    if not model.startswith(RANDOM_PREFIX):
        return load_model(model, dtype=dtype, device=device)[0]
    path, _, seed = model[len(RANDOM_PREFIX):].rpartition(":")
    if not path or not seed.lstrip("-").isdigit():
        raise ValueError(f"--model {model!r}: expected random:<config.json>:<seed>")
    if os.path.isdir(path):
        raw = read_config_json(path)
    else:
        with open(path, "r", encoding="utf-8") as handle:
            raw = json.load(handle)
    _, config = config_from_dict(raw)
    return random_model(config, int(seed), dtype=dtype, device=device)


def replay(model: str, dtype: str, out_dir: str, max_tokens: int | None, lines: IO[str],
           done: IO[str] = sys.stdout, device: str = "cuda:0", block_size: int = DEFAULT_PAGE_TOKENS,
           num_blocks: int | None = None, max_requests: int = DEFAULT_MAX_REQUESTS) -> int:
    """``max_tokens``: the most tokens live requests hold at any time, each request's count rounded up to a
    multiple of 64 (or of the page size, if that is larger); the pool gets just the pages for them, so that
    pages are used again.  ``num_blocks`` sets the pool's size directly instead."""
    if num_blocks is None:
        if max_tokens is None:
            raise ValueError("one of max_tokens and num_blocks is needed to size the cache pool")
        num_blocks = max(1, (int(max_tokens) + block_size - 1) // block_size)
    runner = make_runner(open_model(model, dtype, device), block_size=block_size, num_blocks=int(num_blocks),
                         max_requests=max_requests)
    vocab = runner.vocab_size
    os.makedirs(out_dir, exist_ok=True)
    for line in lines:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        step = record["step"]
        entries, rows = [], []
        for item in record.get("entries", []):
            request_id = item["id"]
            if not runner.cache.has(request_id):
                runner.begin(request_id)
            first = runner.cache.num_tokens(request_id)
            want = [int(w) for w in item.get("want", [])]
            entries.append(StepEntry(request_id, [int(t) for t in item["tokens"]], want))
            rows.extend({"id": request_id, "place": w, "position": first + w} for w in want)
        if entries:
            logits = runner.step(entries)
            if logits.shape[0] > 0:
                host = logits.detach().to("cpu").contiguous().numpy().astype("<f4", copy=False)
                # a small header beside the raw logits: what each row is
                with open(os.path.join(out_dir, f"{step}.json"), "w", encoding="utf-8") as handle:
                    json.dump({"step": step, "dtype": "float32", "byte_order": "little", "shape": [len(rows), vocab],
                               "engine_dtype": dtype, "block_size": block_size, "rows": rows}, handle)
                    handle.write("\n")
                tmp = os.path.join(out_dir, f".{step}.f32.tmp")
                host.tofile(tmp)
                os.replace(tmp, os.path.join(out_dir, f"{step}.f32"))
        for request_id in record.get("end", []):
            if runner.cache.has(request_id):
                runner.end(request_id)
        done.write(f"done {step}\n")
        done.flush()
    return 0
