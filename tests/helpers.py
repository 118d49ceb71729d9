"""Shared by the tests: tiny configurations, traces and comparisons."""

from __future__ import annotations

import os
import random

import torch

from somi_inference_amd.config import Qwen2Config

# Three tiny configurations that differ in every size and option.  A is the reference's own test model
# (tests/conftest.py:27-54 of the reference) with another vocabulary; B has one key/value head, heads of 32, an
# odd vocabulary, an output matrix of its own and other constants; C adds a window on its upper layers, more
# kv heads and sizes that are no power of two.
TINY = {
    "A": dict(config=Qwen2Config(vocab_size=256, hidden_size=64, intermediate_size=128, num_hidden_layers=2,
                                 num_attention_heads=4, num_key_value_heads=2, head_dim=16, rope_theta=10000.0,
                                 rms_norm_eps=1e-6, tie_word_embeddings=True),
              block_size=16, seed=11),
    "B": dict(config=Qwen2Config(vocab_size=503, hidden_size=192, intermediate_size=512, num_hidden_layers=3,
                                 num_attention_heads=6, num_key_value_heads=1, head_dim=32, rope_theta=1e6,
                                 rms_norm_eps=1e-5, tie_word_embeddings=False),
              block_size=8, seed=22),
    "C": dict(config=Qwen2Config(vocab_size=301, hidden_size=120, intermediate_size=200, num_hidden_layers=4,
                                 num_attention_heads=6, num_key_value_heads=3, head_dim=48, rope_theta=5e4,
                                 rms_norm_eps=3e-6, tie_word_embeddings=False, attention_bias=True,
                                 use_sliding_window=True, sliding_window=20, max_window_layers=2),
              block_size=16, seed=33),
}

# float32 engine against the float32 plain implementation: rounding of sums in another order only.
F32_TOL = dict(atol=2e-5, rtol=1e-4)
# bfloat16 engine against the float32 plain implementation (same bfloat16-rounded weights): activations are
# rounded to 8 bits of mantissa (2^-9 relative) at about six places per layer, independently, so the error of
# a logit is a random sum of the order of a per cent of the logits' size, whatever that size is.  Both bounds
# are therefore relative to the logits they are compared with: no element may be off by more than 5 % of the
# largest logit (the share the reference allows half precision, atol = rtol = 5e-2 on values of order one,
# /root/reference/tests/core/test_paged_attention.py:338), and the root mean square error must stay below 3 %
# of the logits' root mean square.  Correct runs of the tests' models measure up to 2.9 % and 1.8 %; a wrong
# key, page or row changes logits by their own size.  The two bounds work as a pair: the element bound alone is
# loose where logits are large (at +-14 it lets a single logit be off by 0.7) and catches single wild values;
# the root mean square bound is the one that bites.  ``per_row`` also holds every row by itself, so that one
# wrong row among hundreds of right ones cannot hide in the mean.  A single row's error spreads more than a
# tensor's: how much rounding a softmax passes on depends on the sequence (over 580 decoded rows of the tests'
# models the rows' errors have a mean of 1.2 % and reach 4.0 %, the same for a request in a batch of 150 as alone
# and whole), so a single row is held to twice the tensor's bound; a row computed from a wrong key, page or
# neighbour is off by about its own size, sixteen times that.
BF16_MAX_SHARE = 5e-2
BF16_RMS_SHARE = 3e-2
BF16_ROW_RMS_SHARE = 6e-2


def write_tiny(name: str, folder: str) -> str:
    from somi_inference_amd.weights import write_random_model
    return write_random_model(folder, TINY[name]["config"], seed=TINY[name]["seed"])


def token_ids(vocab: int, length: int, seed: int) -> list[int]:
    gen = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (length,), generator=gen).tolist()


def assert_close(got: torch.Tensor, want: torch.Tensor, dtype: str, what: str = "", per_row: bool = False) -> None:
    got, want = got.float().cpu(), want.float().cpu()
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} != {tuple(want.shape)}"
    assert bool(torch.isfinite(got).all()), f"{what}: logits that are not finite"
    error = (got - want).abs()
    if dtype == "float32":
        bad = error > F32_TOL["atol"] + F32_TOL["rtol"] * want.abs()
        bound = f"tolerance {F32_TOL}"
    else:
        bad = error > BF16_MAX_SHARE * float(want.abs().max())
        bound = f"bound {BF16_MAX_SHARE} of the largest logit {float(want.abs().max()):.3e}"
    if bad.any():
        row = int(bad.any(dim=-1).nonzero()[0]) if got.dim() == 2 else int(bad.nonzero()[0])
        raise AssertionError(f"{what}: first wrong row {row}, max abs error {error.max():.3e} ({bound})")
    if dtype != "float32":
        rms, size = float(error.pow(2).mean().sqrt()), float(want.pow(2).mean().sqrt())
        assert rms <= BF16_RMS_SHARE * size, f"{what}: root mean square error {rms:.3e} of logits of {size:.3e} (bound {BF16_RMS_SHARE})"
        if per_row and got.dim() == 2:
            row_rms, row_size = error.pow(2).mean(dim=-1).sqrt(), want.pow(2).mean(dim=-1).sqrt()
            over = (row_rms > BF16_ROW_RMS_SHARE * row_size).nonzero().flatten().tolist()
            assert not over, (f"{what}: rows {over[:8]} are off by {[round(float(row_rms[i] / row_size[i]), 4) for i in over[:8]]} "
                              f"of their own size (bound {BF16_ROW_RMS_SHARE} a row)")


def make_engine(folder: str, dtype: str, block_size: int, num_blocks: int, max_requests: int = 8):
    from somi_inference_amd.models import load_model, make_runner
    model, config = load_model(folder, dtype=dtype)
    return make_runner(model, block_size=block_size, num_blocks=num_blocks, max_requests=max_requests), config


def run_portions(runner, request_id, tokens: list[int], sizes: list[int]) -> torch.Tensor:
    """Feed ``tokens`` of one request in portions of the given sizes (cycled), wanting every logit."""
    from somi_inference_amd.engine import StepEntry
    runner.begin(request_id)
    outs, at, i = [], 0, 0
    while at < len(tokens):
        size = max(1, sizes[i % len(sizes)])
        portion = tokens[at:at + size]
        outs.append(runner.step([StepEntry(request_id, portion, list(range(len(portion))))]).cpu())
        at += len(portion)
        i += 1
    runner.end(request_id)
    return torch.cat(outs)


def mixed_trace(requests: dict[str, list[int]], seed: int, max_live: int = 4, portion_sizes=(7, 2, 5, 3, 11, 1)):
    """A schedule over several requests: up to ``max_live`` live at once, prompt portions of changing
    size for some beside single tokens of others, requests ending and new ones starting mid-way.

    Yields steps as ``(entries, ends)`` with entries ``[(id, start, count)]``.
    """
    rng = random.Random(seed)
    pending = list(requests)
    live: dict[str, int] = {}            # id -> tokens fed so far
    steps = []
    while pending or live:
        while pending and len(live) < max_live and (not live or rng.random() < 0.6):
            live[pending.pop(0)] = 0
        entries, ends = [], []
        for rid in list(live):
            if len(live) > 1 and rng.random() < 0.25:
                continue                  # a request may sit a step out
            fed, total = live[rid], len(requests[rid])
            tail = total - min(32, total // 2)       # the last tokens go one by one
            if fed >= tail:
                count = 1
            else:
                count = min(rng.choice(portion_sizes), tail - fed)
                if count == 1 and tail - fed >= 2:
                    count = 2
            entries.append((rid, fed, count))
            live[rid] = fed + count
            if live[rid] == total:
                ends.append(rid)
                del live[rid]
        if entries:
            steps.append((entries, ends))
    return steps


def peaky_folder(source: str, target: str, factor: float = 6.0) -> str:
    """A copy of a model folder whose q and k projections are scaled so that attention scores spread
    over several units: single keys stand out, and a wrong key, page or window edge changes the logits."""
    import shutil
    from safetensors.torch import load_file, save_file
    os.makedirs(target, exist_ok=True)
    shutil.copy(os.path.join(source, "config.json"), os.path.join(target, "config.json"))
    tensors = load_file(os.path.join(source, "model.safetensors"))
    for name in list(tensors):
        if ".q_proj." in name or ".k_proj." in name:
            tensors[name] = (tensors[name].float() * factor).to(tensors[name].dtype)
    save_file(tensors, os.path.join(target, "model.safetensors"))
    return target


def peak_pages(steps, block_size: int) -> int:
    """Most pages live requests hold at any time while a mixed trace runs."""
    held: dict[str, int] = {}
    peak = 0
    for entries, ends in steps:
        for rid, start, count in entries:
            held[rid] = start + count
        peak = max(peak, sum((n + block_size - 1) // block_size for n in held.values()))
        for rid in ends:
            del held[rid]
    return peak
