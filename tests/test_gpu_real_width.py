"""The real width: two layers of the 7B layer sizes under the real vocabulary of 152,064 tokens with an output
matrix of its own, through the entry point, in float32 and in bfloat16, against the plain implementation:
logits at a handful of positions, greedy tokens and a seeded run with a temperature.

The weights are random but shaped so that faults show: q and k are enlarged by 1.5 (single keys stand out
without turning the bfloat16 rounding of q and k into per-cent changes of the attention weights), and the
output matrix by 2.5, so that the logits spread over about +-14 and a distribution at temperature 0.8 has
tokens with a share of several per cent among the 152,064 instead of being flat."""

import json
import os

import pytest
import torch

from helpers import BF16_MAX_SHARE, BF16_RMS_SHARE, assert_close, token_ids
from plain import qwen2_plain as plain
from somi_inference_amd import LLM
from somi_inference_amd.engine import StepEntry
from somi_inference_amd.sampling import uniform

pytestmark = [pytest.mark.gpu, pytest.mark.timeout(900)]     # the fixtures write and read a model of 3 GB
DTYPES = ["float32", "bfloat16"]
VOCAB = 152064
QK_FACTOR, HEAD_FACTOR = 1.5, 2.5
TEMPERATURE, SEED = 0.8, 3


@pytest.fixture(scope="module")
def wide(tmp_path_factory):
    """The model folder, and the plain implementation's weights in float32."""
    from safetensors.torch import load_file, save_file
    from somi_inference_amd.config import Qwen2Config
    from somi_inference_amd.weights import write_random_model
    config = Qwen2Config(vocab_size=VOCAB, hidden_size=3584, intermediate_size=18944, num_hidden_layers=2,
                         num_attention_heads=28, num_key_value_heads=4, head_dim=128, rope_theta=1e6,
                         rms_norm_eps=1e-6, tie_word_embeddings=False)
    folder = str(tmp_path_factory.mktemp("wide") / "two_layers_7b_full_vocabulary")
    print("writing a model of 1.56e9 weights ...", flush=True)
    write_random_model(folder, config, seed=17)
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    for name in list(tensors):
        if ".q_proj." in name or ".k_proj." in name:
            tensors[name] = (tensors[name].float() * QK_FACTOR).to(tensors[name].dtype)
        elif name == "lm_head.weight":
            tensors[name] = (tensors[name].float() * HEAD_FACTOR).to(tensors[name].dtype)
    save_file(tensors, path)
    del tensors
    cfg, weights = plain.read_model(folder)
    assert not cfg["tie_word_embeddings"] and weights["lm_head.weight"].shape == (VOCAB, 3584)
    return folder, cfg, weights


@pytest.fixture(scope="module")
def plain_side(wide):
    """What the plain implementation gives, computed once for both dtypes."""
    _, cfg, weights = wide
    print("plain implementation at the real width ...", flush=True)
    tokens = token_ids(VOCAB, 200, 41)
    places = [0, 1, 15, 16, 63, 64, 150, 199]
    logits = plain.model_logits(cfg, weights, tokens)[places]
    w64 = {k: v.double() for k, v in weights.items()}
    logits64 = plain.model_logits(cfg, w64, tokens)[places]
    del w64
    prompts = [token_ids(VOCAB, n, 50 + n) for n in (37, 6)]
    greedy = [plain.greedy_generate(cfg, weights, p, 5) for p in prompts]
    return dict(tokens=tokens, places=places, logits=logits, logits64=logits64, prompts=prompts, greedy=greedy)


def make_llm(folder, dtype):
    return LLM(folder, dtype=dtype, block_size=16, num_blocks=48, max_concurrent=4, eos_token_id=-1)


@pytest.mark.parametrize("dtype", DTYPES)
def test_logits_at_a_handful_of_positions(dtype, wide, plain_side):
    folder, _, _ = wide
    llm = make_llm(folder, dtype)
    tokens, places = plain_side["tokens"], plain_side["places"]
    runner = llm.runner
    runner.begin("whole")
    got = runner.step([StepEntry("whole", tokens, places)]).cpu()
    runner.end("whole")
    assert got.shape == (len(places), VOCAB)
    want, want64 = plain_side["logits"], plain_side["logits64"]
    assert float(want.abs().max()) > 10.0 and float(want.std()) > 2.0, "the logits do not spread as the test means them to"
    if dtype == "float32":
        # sums over 3,584 to 18,944 terms: the engine is held to the plain float32 implementation's own accuracy,
        # both measured against the plain implementation in float64
        plain_error = float((want.double() - want64).abs().max())
        error = float((got.double() - want64).abs().max())
        assert error <= 4 * plain_error + 1e-6, f"error {error:.3e}, the plain float32 implementation's {plain_error:.3e}"
    else:
        assert_close(got, want, dtype, "bfloat16 at the real width", per_row=True)
    # the same places when the prompt comes in portions and its last 32 tokens one by one
    runner.begin("cut")
    rows, at = [], 0
    for size in [100, 2, 66] + [1] * 32:
        inside = [p - at for p in places if at <= p < at + size]
        out = runner.step([StepEntry("cut", tokens[at:at + size], inside)])
        if inside:
            rows.append(out.cpu())
        at += size
    runner.end("cut")
    cut = torch.cat(rows)
    if dtype == "float32":
        error = float((cut.double() - want64).abs().max())
        assert error <= 4 * plain_error + 1e-6, f"in portions: error {error:.3e}, plain float32 {plain_error:.3e}"
    else:
        assert_close(cut, want, dtype, "bfloat16 at the real width, in portions", per_row=True)
    assert llm.kv_manager.free_pages() == [48]


@pytest.mark.parametrize("dtype", DTYPES)
def test_greedy_and_seeded_temperature_generation(dtype, wide, plain_side):
    folder, cfg, weights = wide
    llm = make_llm(folder, dtype)
    prompts = plain_side["prompts"]
    got = llm.generate(prompts, max_new_tokens=5, temperature=0.0)
    for prompt, tokens, expected in zip(prompts, got, plain_side["greedy"]):
        if tokens == expected:
            continue
        assert dtype != "float32", f"float32 tokens {tokens} differ from the plain implementation's {expected}"
        # bfloat16 may take another token only where the plain logits of the two nearly tie: within twice the
        # error a single bfloat16 logit may have
        first = next(i for i, (a, b) in enumerate(zip(tokens, expected)) if a != b)
        logits = plain.model_logits(cfg, weights, prompt + expected[:first])[-1]
        gap = float(logits[expected[first]] - logits[tokens[first]])
        assert 0.0 <= gap <= 2 * BF16_MAX_SHARE * float(logits.abs().max()), \
            f"token {tokens[first]} instead of {expected[first]} at {first}: gap {gap}"

    # one run with a temperature and a seed: request i draws its n-th token at uniform(seed + i, n) from the
    # plain implementation's distribution of what the engine itself produced so far
    sampled = llm.generate(prompts, max_new_tokens=4, temperature=TEMPERATURE, seed=SEED)
    assert sampled == llm.generate(prompts, max_new_tokens=4, temperature=TEMPERATURE, seed=SEED)
    assert sampled != [g[:4] for g in got]
    heavy = 0
    for index, (prompt, tokens) in enumerate(zip(prompts, sampled)):
        for n, token in enumerate(tokens):
            logits = plain.model_logits(cfg, weights, prompt + tokens[:n])[-1]
            share = plain.sampling_distribution(logits, [], TEMPERATURE).double()
            cdf = torch.cumsum(share, dim=0)
            # bfloat16 logits are off by up to about BF16_RMS_SHARE of their root mean square; over the temperature,
            # that is the share of probability mass that may lie on the other side of an edge of the distribution
            slack = 1e-4 if dtype == "float32" else BF16_RMS_SHARE * float(logits.pow(2).mean().sqrt()) / TEMPERATURE
            u = uniform(SEED + index, n)
            low = float(cdf[token - 1]) if token > 0 else 0.0
            assert low - slack <= u <= float(cdf[token]) + slack, \
                f"prompt {index}, draw {n}: token {token} covers [{low:.5f}, {float(cdf[token]):.5f}], drawn at {u:.5f}"
            heavy += int(float(share.max()) > 0.02)
    assert heavy >= 4, "the distributions are flat: a draw says little about the logits"
    assert llm.kv_manager.free_pages() == [48]
    json.dumps(sampled)      # plain lists of ints


def test_many_requests_decode_together_at_the_real_width(wide):
    """150 and 260 requests in one decode step in bfloat16: at these widths the products into the stream and the
    q/k/v product share a tile's K among workgroups, and the logits of all rows come from one pass over the output
    matrix.  The logits of every request against the plain implementation, each row with its own bounds."""
    folder, cfg, weights = wide
    llm = LLM(folder, dtype="bfloat16", block_size=16, num_blocks=300, max_concurrent=270, eos_token_id=-1)
    runner = llm.runner
    for batch in (150, 260):
        ids = [f"w{batch}_{i}" for i in range(batch)]
        tokens = [token_ids(VOCAB, 2 + (i * 5) % 11, 900 + batch + i) for i in range(batch)]
        for rid, prompt in zip(ids, tokens):
            runner.begin(rid)
            runner.step([StepEntry(rid, prompt[:-1], [])])
        for step in range(2):
            logits = runner.step([StepEntry(rid, [seq[-1]], [0]) for rid, seq in zip(ids, tokens)])
            if step == 0:
                for seq, token in zip(tokens, logits.argmax(dim=-1).tolist()):
                    seq.append(int(token))
        logits = logits.cpu()
        assert logits.shape == (batch, VOCAB) and logits.dtype == torch.float32
        want = torch.cat([plain.model_logits(cfg, weights, tokens[i], rows=[len(tokens[i]) - 1]) for i in range(batch)])
        assert_close(logits, want, "bfloat16", f"{batch} requests after 2 to 13 tokens", per_row=True)
        for rid in ids:
            runner.end(rid)
    assert llm.kv_manager.free_pages() == [300]
