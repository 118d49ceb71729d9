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

from ..engine.batch import StepEntry
from ..models.loader import load_model, make_runner

PAGE_TOKENS = 16          # tokens per cache page; divides the 64 that --max-tokens is counted in
MAX_LIVE_REQUESTS = 64


def replay(model_dir: str, dtype: str, out_dir: str, max_tokens: int, lines: IO[str],
           done: IO[str] = sys.stdout, device: str = "cuda:0", block_size: int = PAGE_TOKENS) -> int:
    model, _ = load_model(model_dir, dtype=dtype, device=device)
    num_blocks = max(1, (int(max_tokens) + block_size - 1) // block_size)
    runner = make_runner(model, block_size=block_size, num_blocks=num_blocks, max_requests=MAX_LIVE_REQUESTS)
    os.makedirs(out_dir, exist_ok=True)
    for line in lines:
        line = line.strip()
        if not line:
            continue
        record = json.loads(line)
        step = record["step"]
        entries = []
        for item in record.get("entries", []):
            request_id = item["id"]
            if not runner.cache.has(request_id):
                runner.begin(request_id)
            entries.append(StepEntry(request_id, [int(t) for t in item["tokens"]],
                                     [int(w) for w in item.get("want", [])]))
        if entries:
            logits = runner.step(entries)
            if logits.shape[0] > 0:
                host = logits.detach().to("cpu").contiguous().numpy().astype("<f4", copy=False)
                tmp = os.path.join(out_dir, f".{step}.f32.tmp")
                host.tofile(tmp)
                os.replace(tmp, os.path.join(out_dir, f"{step}.f32"))
        for request_id in record.get("end", []):
            if runner.cache.has(request_id):
                runner.end(request_id)
        done.write(f"done {step}\n")
        done.flush()
    return 0
