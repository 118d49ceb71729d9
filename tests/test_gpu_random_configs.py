"""Random tiny configurations (head counts and groups, head sizes in steps of 16 and two that are not, widths
and vocabularies that are no power of two, windows, page sizes) under random mixed traces with so few pages
that they are used again: the engine against the plain implementation, in float32 and bfloat16."""

import os
import random

import pytest
import torch

from helpers import assert_close, make_engine, mixed_trace, peak_pages, peaky_folder, token_ids
from plain import qwen2_plain as plain
from somi_inference_amd.config import Qwen2Config
from somi_inference_amd.engine import StepEntry
from somi_inference_amd.weights import write_random_model

pytestmark = pytest.mark.gpu


def random_case(seed: int, odd: bool = False):
    """``odd``: widths that are no multiple of 8 and head sizes that are no multiple of 16 or beyond 128, which
    take the plain kernels in places."""
    rng = random.Random(seed + (1000 if odd else 0))
    nkv = rng.choice([1, 2, 3, 4, 5])
    nq = nkv * rng.choice([1, 2, 3, 4, 7, 8])
    layers = rng.choice([1, 2, 3])
    window = rng.random() < 0.4
    config = Qwen2Config(
        vocab_size=rng.choice([97, 256, 301, 503, 1000]),
        hidden_size=rng.choice([36, 50, 66, 100, 44, 68] if odd else [40, 64, 72, 120, 136, 200]),
        intermediate_size=rng.choice([50, 70, 100, 36, 132] if odd else [48, 96, 160, 200, 272, 520]),
        num_hidden_layers=layers, num_attention_heads=nq, num_key_value_heads=nkv,
        head_dim=rng.choice([6, 10, 18, 24, 40, 144, 160, 256] if odd else [16, 32, 48, 64, 80, 96, 112, 128, 24, 40]),
        rope_theta=rng.choice([1e4, 5e4, 1e6]), rms_norm_eps=rng.choice([1e-6, 1e-5, 3e-6]),
        tie_word_embeddings=rng.random() < 0.5, attention_bias=rng.random() < 0.8,
        use_sliding_window=window, sliding_window=rng.choice([5, 20, 33, 64]) if window else None,
        max_window_layers=rng.randrange(0, layers) if window else None)
    block_size = rng.choice([4, 8, 12, 16, 32, 64])
    return rng, config, block_size


@pytest.mark.parametrize("odd", [False, True], ids=["even", "odd"])
@pytest.mark.parametrize("seed", range(40))
def test_random_configuration_under_a_random_mixed_trace(seed, odd, tmp_path):
    rng, config, block_size = random_case(seed, odd)
    base = write_random_model(str(tmp_path / "model"), config, seed=rng.randrange(1000))
    folder = peaky_folder(base, str(tmp_path / "peaky"), factor=rng.choice([1.0, 3.0, 4.0]))
    plain_config, weights = plain.read_model(folder)
    lengths = {f"r{i}": rng.choice([2, 3, 17, 33, 45, 64, 70, 100, 129, 200]) for i in range(rng.randrange(3, 7))}
    requests = {rid: token_ids(config.vocab_size, n, rng.randrange(10000)) for rid, n in lengths.items()}
    sizes = tuple(rng.choice([1, 2, 3, 5, 7, 8, 9, 11, 16, 17, 31, 64, 65]) for _ in range(6))
    steps = mixed_trace(requests, seed=rng.randrange(1000), portion_sizes=sizes)
    pages = peak_pages(steps, block_size)
    want = {rid: plain.model_logits(plain_config, weights, tokens) for rid, tokens in requests.items()}
    for dtype in ("float32", "bfloat16"):
        runner, _ = make_engine(folder, dtype, block_size, pages, max_requests=4)
        rows = {rid: [] for rid in requests}
        for entries, ends in steps:
            batch = []
            for rid, start, count in entries:
                if not runner.cache.has(rid):
                    runner.begin(rid)
                batch.append(StepEntry(rid, requests[rid][start:start + count], list(range(count))))
            logits = runner.step(batch).cpu()
            at = 0
            for rid, start, count in entries:
                rows[rid].append(logits[at:at + count])
                at += count
            for rid in ends:
                runner.end(rid)
            runner.cache.check_invariants()
        what = f"seed {seed} {dtype} {config} pages of {block_size}"
        for rid, tokens in requests.items():
            mixed = torch.cat(rows[rid])
            assert_close(mixed, want[rid], dtype, f"{what}: request {rid} of {lengths[rid]} in a mixed trace")
            if dtype == "float32":
                runner.begin("whole")
                whole = runner.step([StepEntry("whole", tokens, list(range(len(tokens))))]).cpu()
                runner.end("whole")
                assert torch.equal(mixed, whole), f"{what}: float32 logits of {rid} depend on the cutting"
        assert runner.cache.free_pages() == [pages] * len(runner.cache.groups)
