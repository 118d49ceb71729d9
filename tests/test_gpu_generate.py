"""Generation through the entry point and the command line: greedy against the plain implementation,
temperature sampling with a request's own seed, sampler rules on the GPU, and what happens when pages run out."""

import json
import os
import subprocess
import sys

import pytest
import torch

from helpers import TINY, token_ids
from plain import qwen2_plain as plain
from somi_inference_amd import LLM, SamplingParams
from somi_inference_amd.sampling import Sampler, uniform

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def plain_greedy(folder, prompts, new_tokens):
    cfg, weights = plain.read_model(folder)
    return [plain.greedy_generate(cfg, weights, p, new_tokens) for p in prompts], cfg, weights


def assert_greedy_matches(got, want, prompts, cfg, weights, exact):
    for prompt, tokens, expected in zip(prompts, got, want):
        if tokens == expected:
            continue
        assert not exact, f"float32 tokens {tokens} differ from the plain implementation's {expected}"
        first = next(i for i, (a, b) in enumerate(zip(tokens, expected)) if a != b)
        logits = plain.model_logits(cfg, weights, prompt + expected[:first])[-1]
        gap = float(logits[expected[first]] - logits[tokens[first]])
        assert 0.0 <= gap < 0.03, f"token {tokens[first]} instead of {expected[first]} at {first}: gap {gap}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_of_the_small_workload(dtype, model_folders):
    # prompts of 5, 17 and 33 tokens, 8 greedy tokens each, pages of 16
    vocab = TINY["A"]["config"].vocab_size
    prompts = [token_ids(vocab, n, 10 + n) for n in (5, 17, 33)]
    want, cfg, weights = plain_greedy(model_folders["A"], prompts, 8)
    llm = LLM(model_folders["A"], dtype=dtype, block_size=16, num_blocks=16, max_concurrent=4, eos_token_id=-1)
    got = llm.generate(prompts, max_new_tokens=8, temperature=0.0)
    assert_greedy_matches(got, want, prompts, cfg, weights, exact=dtype == "float32")
    assert llm.kv_manager.free_pages() == [16]
    one = llm.generate(prompts[0], max_new_tokens=8, temperature=0.0)       # a single prompt gives a single result
    assert one == got[0]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prompts_in_portions_of_seven_beside_decoding(dtype, model_folders):
    # prompts of 1, 9, 40, 64 and 100 tokens, 12 tokens each, portions of 7 mixed with decoded tokens, pages of 8
    vocab = TINY["B"]["config"].vocab_size
    prompts = [token_ids(vocab, n, 20 + n) for n in (1, 9, 40, 64, 100)]
    want, cfg, weights = plain_greedy(model_folders["B"], prompts, 12)
    llm = LLM(model_folders["B"], dtype=dtype, block_size=8, num_blocks=64, max_concurrent=5,
              max_num_batched_tokens=24, max_chunk=7, eos_token_id=-1)
    got = llm.generate(prompts, max_new_tokens=12, temperature=0.0)
    assert_greedy_matches(got, want, prompts, cfg, weights, exact=dtype == "float32")
    assert llm.engine.num_steps > 12                       # the prompts really were cut up
    # temperature 0.8 with a fixed seed: the same tokens whatever the batch and the portions are
    sampled = llm.generate(prompts, max_new_tokens=12, temperature=0.8, seed=5)
    alone = LLM(model_folders["B"], dtype=dtype, block_size=8, num_blocks=64, max_concurrent=1, eos_token_id=-1)
    for index, prompt in enumerate(prompts):
        if dtype == "float32":
            assert alone.generate(prompt, max_new_tokens=12, temperature=0.8, seed=5 + index) == sampled[index]
    assert sampled != got
    assert llm.generate(prompts, max_new_tokens=12, temperature=0.8, seed=5) == sampled


def assert_sampled_matches(got, want, prompts, cfg, weights, temperature, seed, exact):
    """Tokens drawn with a temperature by two runs that cut or batch the work differently.  The float32 engine
    must give the same tokens.  In bfloat16 the two runs' logits differ by rounding, so a draw may fall on the
    other side of an edge of the cumulative distribution: at the first difference, both tokens must lie within
    2 % of probability mass of the request's uniform number in the plain implementation's distribution."""
    for index, (prompt, tokens, expected) in enumerate(zip(prompts, got, want)):
        if tokens == expected:
            continue
        assert not exact, f"float32 tokens {tokens} differ from {expected}"
        first = next(i for i, (a, b) in enumerate(zip(tokens, expected)) if a != b)
        logits = plain.model_logits(cfg, weights, prompt + expected[:first])[-1]
        cdf = torch.cumsum(plain.sampling_distribution(logits, [], temperature).double(), dim=0)
        u = uniform(seed + index, first)
        for token in (tokens[first], expected[first]):
            low = float(cdf[token - 1]) if token > 0 else 0.0
            assert low - 0.02 <= u <= float(cdf[token]) + 0.02, \
                f"prompt {index}, token {first}: {token} covers [{low:.4f}, {float(cdf[token]):.4f}], drawn at {u:.4f}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_running_out_of_pages_preempts_and_still_gives_the_same_tokens(dtype, model_folders):
    vocab = TINY["A"]["config"].vocab_size
    prompts = [token_ids(vocab, n, 30 + n) for n in (30, 28, 25)]
    cfg, weights = plain.read_model(model_folders["A"])
    roomy = LLM(model_folders["A"], dtype=dtype, block_size=16, num_blocks=32, max_concurrent=3, eos_token_id=-1)
    want = roomy.generate(prompts, max_new_tokens=24, temperature=0.7, seed=1)
    tight = LLM(model_folders["A"], dtype=dtype, block_size=16, num_blocks=7, max_concurrent=3, eos_token_id=-1)
    got = tight.generate(prompts, max_new_tokens=24, temperature=0.7, seed=1)
    assert_sampled_matches(got, want, prompts, cfg, weights, 0.7, 1, exact=dtype == "float32")
    assert tight.kv_manager.free_pages() == [7]
    tight.kv_manager.check_invariants()
    assert tight.scheduler.preemptions > 0 and roomy.scheduler.preemptions == 0


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_temperature_sampling_does_not_depend_on_the_batch(dtype, model_folders):
    """A request's draws come from its own seed and token count: alone, or in portions of 7 beside four others,
    it gets the same tokens (in bfloat16 up to draws that sit on an edge of the distribution)."""
    vocab = TINY["B"]["config"].vocab_size
    prompts = [token_ids(vocab, n, 20 + n) for n in (1, 9, 40, 64, 100)]
    cfg, weights = plain.read_model(model_folders["B"])
    together = LLM(model_folders["B"], dtype=dtype, block_size=8, num_blocks=64, max_concurrent=5,
                   max_num_batched_tokens=24, max_chunk=7, eos_token_id=-1)
    sampled = together.generate(prompts, max_new_tokens=12, temperature=0.8, seed=5)
    alone = LLM(model_folders["B"], dtype=dtype, block_size=8, num_blocks=64, max_concurrent=1, eos_token_id=-1)
    single = [alone.generate(prompt, max_new_tokens=12, temperature=0.8, seed=5 + index)
              for index, prompt in enumerate(prompts)]
    assert_sampled_matches(sampled, single, prompts, cfg, weights, 0.8, 5, exact=dtype == "float32")
    # and they are draws from the plain implementation's distribution, not just equal to each other
    for index, (prompt, tokens) in enumerate(zip(prompts, single)):
        logits = plain.model_logits(cfg, weights, prompt)[-1]
        cdf = torch.cumsum(plain.sampling_distribution(logits, [], 0.8).double(), dim=0)
        u, token = uniform(5 + index, 0), tokens[0]
        low = float(cdf[token - 1]) if token > 0 else 0.0
        slack = 1e-5 if dtype == "float32" else 0.02
        assert low - slack <= u <= float(cdf[token]) + slack


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_repetition_penalty_top_k_and_top_p_through_generate_follow_the_plain_rules(dtype, model_folders):
    """Generation through the entry point with a repetition penalty (which reads each request's history, prompt
    and outputs: /root/reference/somi_inference/core/continuous_batching.py:167, core/model_runner.py:36, and so
    keeps the engine from running ahead), alone and with a temperature, top-k and top-p, in portions beside
    decoding requests.  Every token of every request is held against the plain rules applied to the plain logits
    of what the engine produced so far: the greedy token is the argmax of the penalised logits, a drawn token is
    the one whose share of the plain distribution (penalty, temperature, top-k, top-p, softmax) covers the
    request's uniform number."""
    vocab = TINY["B"]["config"].vocab_size
    prompts = [token_ids(vocab, n, 80 + n) for n in (4, 23, 40, 64, 100)]
    cfg, weights = plain.read_model(model_folders["B"])
    llm = LLM(model_folders["B"], dtype=dtype, block_size=8, num_blocks=96, max_concurrent=5,
              max_num_batched_tokens=40, max_chunk=13, eos_token_id=-1)
    exact = dtype == "float32"
    penalty, new_tokens = 1.3, 16

    greedy = llm.generate(prompts, max_new_tokens=new_tokens, temperature=0.0, repetition_penalty=penalty)
    assert llm.engine.steps_run_ahead == 0 and llm.engine.num_steps > new_tokens
    moved = 0
    for index, (prompt, tokens) in enumerate(zip(prompts, greedy)):
        assert len(tokens) == new_tokens
        for n, token in enumerate(tokens):
            history = prompt + tokens[:n]
            logits = plain.model_logits(cfg, weights, history, rows=[len(history) - 1])[0]
            ruled = plain.penalize_repetition(logits, history, penalty)
            want = int(torch.argmax(ruled))
            moved += int(want != int(torch.argmax(logits)))
            if token != want:
                assert not exact, f"prompt {index}, token {n}: {token} instead of {want}"
                gap = float(ruled[want] - ruled[token])
                assert 0.0 <= gap < 0.03, f"prompt {index}, token {n}: {token} instead of {want}, gap {gap}"
    assert moved >= 5, "the penalty never changed the choice: the test says nothing about it"
    unruled = llm.generate(prompts, max_new_tokens=new_tokens, temperature=0.0)
    assert unruled != greedy

    heavy = 0
    for options in (dict(temperature=0.7, top_p=0.9), dict(temperature=0.9, top_k=12, top_p=0.8)):
        seed = 31
        drawn = llm.generate(prompts, max_new_tokens=new_tokens, repetition_penalty=penalty, seed=seed, **options)
        assert drawn == llm.generate(prompts, max_new_tokens=new_tokens, repetition_penalty=penalty, seed=seed, **options)
        for index, (prompt, tokens) in enumerate(zip(prompts, drawn)):
            for n, token in enumerate(tokens):
                history = prompt + tokens[:n]
                logits = plain.model_logits(cfg, weights, history, rows=[len(history) - 1])[0]
                share = plain.sampling_distribution(logits, history, options["temperature"], options.get("top_k", -1),
                                                    options["top_p"], penalty).double()
                cdf = torch.cumsum(share, dim=0)
                u = uniform(seed + index, n)
                low = float(cdf[token - 1]) if token > 0 else 0.0
                # float32 holds the rules exactly.  bfloat16 logits differ by rounding: beside the 2 % of mass that
                # may lie on the other side of an interval's edge, the entry at the edge of what top-k / top-p keep
                # may fall on the other side of the cut, which rescales the cumulative sums by that entry's share
                # (m / (1 - m) at the far end)
                edge = float(share[share > 0].min())
                slack = 1e-5 if exact else 0.02 + 1.5 * edge
                assert low - slack <= u <= float(cdf[token]) + slack, \
                    f"{options}, prompt {index}, draw {n}: token {token} covers [{low:.5f}, {float(cdf[token]):.5f}], drawn at {u:.5f}"
                if exact:
                    assert float(share[token]) > 0.0, f"{options}: token {token} lies outside what top-k / top-p keep"
                heavy += int(int((share > 0).sum()) < vocab // 2)
    assert heavy > 0, "top-k / top-p never cut anything away"
    assert llm.kv_manager.free_pages() == [96]
    llm.kv_manager.check_invariants()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_generation_of_the_windowed_configuration(dtype, model_folders):
    """Layers with a window of 20 keys beside layers that see everything: greedy tokens through the entry point
    (scheduler, captured decode steps, running ahead) against the plain implementation, with prompts shorter and
    longer than the window and portions that straddle it; the window's pages come back while requests run."""
    vocab = TINY["C"]["config"].vocab_size
    prompts = [token_ids(vocab, n, 60 + n) for n in (3, 19, 21, 47, 90)]
    want, cfg, weights = plain_greedy(model_folders["C"], prompts, 30)
    llm = LLM(model_folders["C"], dtype=dtype, block_size=16, num_blocks=40, max_concurrent=5,
              max_num_batched_tokens=40, max_chunk=13, eos_token_id=-1)
    assert len(llm.kv_manager.groups) == 2
    got = llm.generate(prompts, max_new_tokens=30, temperature=0.0)
    assert_greedy_matches(got, want, prompts, cfg, weights, exact=dtype == "float32")
    assert llm.kv_manager.free_pages() == [40, 40]
    llm.kv_manager.check_invariants()
    assert llm.engine.steps_run_ahead > 0


def test_a_step_whose_forward_raises_gives_its_pages_back(model_folders):
    from somi_inference_amd.engine import StepEntry
    llm = LLM(model_folders["A"], dtype="bfloat16", block_size=16, num_blocks=8, max_concurrent=2, eos_token_id=-1)
    runner, cache = llm.runner, llm.kv_manager
    runner.begin("r")
    runner.step([StepEntry("r", list(range(10)), [9])])
    free = cache.free_pages()
    forward = runner.model.forward

    def failing(batch, caches):
        raise RuntimeError("a kernel refused its arguments")
    runner.model.forward = failing
    with pytest.raises(RuntimeError, match="refused"):
        runner.step([StepEntry("r", list(range(30)), [])])          # two more pages reserved, none committed
    runner.model.forward = forward
    assert cache.free_pages() == free and cache.num_tokens("r") == 10
    cache.check_invariants()
    again = runner.step([StepEntry("r", list(range(30)), [29])])    # and the request goes on from where it stood
    assert again.shape[0] == 1 and cache.num_tokens("r") == 40
    runner.end("r")
    # through the entry point: the call's requests are aborted, the next call runs
    calls = {"n": 0}

    def failing_later(batch, caches):
        calls["n"] += 1
        if calls["n"] == 3:
            raise RuntimeError("a kernel refused its arguments")
        return forward(batch, caches)
    runner.model.forward = failing_later
    runner.decode_graphs = False
    prompts = [list(range(5, 25)), list(range(40, 47))]
    with pytest.raises(RuntimeError, match="refused"):
        llm.generate(prompts, max_new_tokens=6, temperature=0.0)
    runner.model.forward = forward
    assert cache.free_pages() == [8] and not cache.live_requests()
    want, cfg, weights = plain_greedy(model_folders["A"], prompts, 6)
    assert_greedy_matches(llm.generate(prompts, max_new_tokens=6, temperature=0.0), want, prompts, cfg, weights, exact=False)


def test_eos_ends_a_request_and_is_kept(model_folders):
    vocab = TINY["A"]["config"].vocab_size
    prompt = token_ids(vocab, 9, 3)
    free = LLM(model_folders["A"], dtype="float32", num_blocks=8, eos_token_id=-1).generate(prompt, max_new_tokens=6, temperature=0.0)
    eos = free[2]
    stopped = LLM(model_folders["A"], dtype="float32", num_blocks=8, eos_token_id=eos).generate(prompt, max_new_tokens=6, temperature=0.0)
    assert stopped == free[:free.index(eos) + 1]


def test_entry_point_options_and_errors(model_folders):
    llm = LLM(model_folders["A"], num_blocks=4)
    assert llm.dtype == "float32"                            # the reference's default dtype (entrypoints/llm.py:66)
    with pytest.raises(NotImplementedError):                 # reference entrypoints/llm.py:166-170
        llm.generate_stream("x", max_new_tokens=1)
    with pytest.raises(ValueError, match="tokenizer"):
        llm.generate("some text", max_new_tokens=1)
    with pytest.raises(ValueError, match="max_new_tokens"):
        llm.generate([1, 2], max_new_tokens=0)
    with pytest.raises(ValueError, match="pages"):
        llm.generate(list(range(60)), max_new_tokens=10)
    with pytest.raises(RuntimeError, match="GPU"):
        LLM(model_folders["A"], device="cpu")


def test_page_pool_sized_by_the_free_memory(model_folders):
    from somi_inference_amd.cache import CacheManager
    fixed = LLM(model_folders["B"], dtype="bfloat16", num_blocks=64, block_size=8)
    free, _ = torch.cuda.mem_get_info()
    sized = LLM(model_folders["B"], dtype="bfloat16", num_blocks=None, memory_fraction=0.001, block_size=8)
    per_page = CacheManager.page_bytes(sized.model.cache_needs(), 8, torch.bfloat16)
    cfg = TINY["B"]["config"]
    assert per_page == cfg.num_hidden_layers * 2 * cfg.num_key_value_heads * cfg.head_dim * 8 * 2
    pages = sized.kv_manager.num_blocks
    assert pages == sized.options.num_blocks and 0.5 * free * 0.001 / per_page < pages <= free * 0.001 / per_page
    prompts = [token_ids(cfg.vocab_size, n, 70 + n) for n in (9, 40)]
    assert sized.generate(prompts, max_new_tokens=6, temperature=0.0) == fixed.generate(prompts, max_new_tokens=6, temperature=0.0)
    with pytest.raises(ValueError, match="memory_fraction"):
        LLM(model_folders["B"], dtype="bfloat16", num_blocks=None, memory_fraction=0.0)


def test_sampler_rules_on_the_gpu():
    sampler, dev = Sampler(), "cuda:0"
    t = lambda rows: torch.tensor(rows, dtype=torch.float32, device=dev)
    greedy = SamplingParams(temperature=0.0)
    assert sampler.sample(t([[1.0, 3.0, 2.0]]), greedy) == [1]                                     # reference test_sampler.py:58-66
    assert sampler.sample(t([[2.0, 1.5]]), SamplingParams(temperature=0.0, repetition_penalty=2.0), [[0]]) == [1]   # :85-93
    assert sampler.sample(t([[-1.0, 0.5, 0.5]]), SamplingParams(temperature=0.0, repetition_penalty=2.0), [[0]])[0] != 0
    rows = t([[1.0, 2.9, 3.0], [1.0, 2.9, 3.0]])
    assert sampler.sample(rows, SamplingParams(temperature=0.0, repetition_penalty=1.5), [[2], [1]]) == [1, 2]     # :251-279
    # temperature 0 ignores top-k and top-p (:131-141)
    assert sampler.sample(t([[1.0, 5.0, 2.0]]), SamplingParams(temperature=0.0, top_k=1, top_p=0.1)) == [1]
    # top-k keeps exactly k also under ties; top-p keeps the entry that crosses p (:96-128)
    for counter in range(50):
        picked = sampler.sample(t([[5.0, 4.0, 4.0, 1.0]]), SamplingParams(top_k=2), seeds=[3], counters=[counter])[0]
        assert picked in (0, 1, 2) and picked != 3
        assert sampler.sample(t([[4.0, 3.0, 2.0, 1.0]]), SamplingParams(top_p=0.5), seeds=[3], counters=[counter]) == [0]
    # heterogeneous rows in one call (:144-160), and the caller's logits are not modified
    logits = t([[0.0, 9.0, 1.0], [3.0, 1.0, 2.0]])
    keep = logits.clone()
    out = sampler.sample(logits, [SamplingParams(temperature=0.0), SamplingParams(top_k=1, repetition_penalty=3.0)], [[], [1]])
    assert out == [1, 0] and torch.equal(logits, keep)
    # the draws follow the softmax: frequencies over the request's own stream
    probs = torch.softmax(t([1.0, 2.0, 0.5, 3.0]) / 0.8, dim=-1).cpu()
    n = 3000
    rows = t([[1.0, 2.0, 0.5, 3.0]]).expand(n, -1).contiguous()
    picks = torch.tensor(sampler.sample(rows, SamplingParams(temperature=0.8), seeds=[11] * n, counters=list(range(n))))
    freq = torch.bincount(picks, minlength=4).float() / n
    assert (freq - probs).abs().max() < 0.03
    assert 0.0 <= uniform(1, 2) < 1.0 and uniform(1, 2) == uniform(1, 2) != uniform(1, 3)


def test_command_line_generates_and_appends_jsonl(model_folders, tmp_path):
    vocab = TINY["A"]["config"].vocab_size
    prompt = token_ids(vocab, 6, 1)
    out_file = tmp_path / "out.jsonl"
    cmd = [sys.executable, "-m", "somi_inference_amd.entrypoints.cli", "--model-name", model_folders["A"],
           "--dtype", "float32", "--num-blocks", "8", "--max-new-tokens", "5", "--temperature", "0.0",
           "--prompt-ids", ",".join(map(str, prompt)), "--output-file", str(out_file)]
    done = subprocess.run(cmd, cwd=ROOT, capture_output=True, text=True, timeout=300)
    assert done.returncode == 0, done.stderr[-2000:]
    record = json.loads(done.stdout.strip().splitlines()[-1])
    cfg, weights = plain.read_model(model_folders["A"])
    want = plain.greedy_generate(cfg, weights, prompt, 5, eos=cfg.get("eos_token_id"))
    assert record["prompt"] == prompt and record["output"] == want
    assert json.loads(out_file.read_text().strip()) == record


def test_warm_up_captures_decode_graphs_without_changing_results(model_folders, tmp_path, monkeypatch):
    """The optional warm-up captures the decode graphs ahead of any request: the tokens stay what the plain
    implementation gives, the pages are all given back, generation captures no graph of its own, and no file
    appears in the working directory."""
    monkeypatch.chdir(tmp_path)
    folder = model_folders["B"]
    llm = LLM(folder, dtype="bfloat16", num_blocks=64, block_size=8, max_num_batched_tokens=96, max_concurrent=4,
              eos_token_id=-1)
    free_before = llm.kv_manager.free_pages()
    # up to 4 requests (1, 2 and 4 rows) with tables of 16, 32 and 64 pages (the pool's 512 tokens)
    assert llm.warm_up() == 9
    assert sorted(llm.runner._graphs) == [(rows, (width,)) for rows in (1, 2, 4) for width in (16, 32, 64)]
    assert llm.kv_manager.free_pages() == free_before
    llm.kv_manager.check_invariants()
    prompts = [token_ids(TINY["B"]["config"].vocab_size, 96, 3)]
    want, cfg, weights = plain_greedy(folder, prompts, 6)
    got = llm.generate(prompts, max_new_tokens=6, temperature=0.0)
    assert_greedy_matches(got, want, prompts, cfg, weights, exact=False)
    assert len(llm.runner._graphs) == 9 and llm.runner.graph_replays > 0, "generation captured a graph of its own"
    assert list(tmp_path.iterdir()) == []
    assert LLM(folder, dtype="float32", num_blocks=64, block_size=8, max_concurrent=2).warm_up() == 6


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_running_ahead_of_the_device_gives_the_same_tokens(dtype, model_folders):
    """While only decoding requests run, the engine launches step n + 1 before it has read step n's tokens.
    With it switched off the same tokens come out: greedy and with temperature, with requests of different
    lengths (so that some end while others go on) and with an end-of-sequence token that really occurs (so
    that a request has run one token too far when the host finds out)."""
    vocab = TINY["B"]["config"].vocab_size
    prompts = [token_ids(vocab, n, 40 + n) for n in (3, 18, 33, 7)]

    def run(ahead, **options):
        llm = LLM(model_folders["B"], dtype=dtype, block_size=8, num_blocks=64, max_concurrent=4, **options)
        llm.engine.run_ahead = ahead
        out = [llm.generate(prompts, max_new_tokens=24, temperature=0.0),
               llm.generate(prompts, max_new_tokens=24, temperature=0.9, top_k=20, seed=11),
               llm.generate(prompts[:2], max_new_tokens=5, temperature=0.0) + llm.generate(prompts[2:], max_new_tokens=9, temperature=0.0)]
        assert llm.kv_manager.free_pages() == [64]
        llm.kv_manager.check_invariants()
        return out, llm.engine.steps_run_ahead

    want, none_ahead = run(False, eos_token_id=-1)
    got, some_ahead = run(True, eos_token_id=-1)
    assert none_ahead == 0 and some_ahead > 40
    assert got == want
    assert all(len(tokens) == 24 and min(tokens) >= 0 for tokens in got[0])
    # an end-of-sequence token that occurs in the middle of the first request's greedy tokens
    eos = want[0][0][10]
    want_eos, _ = run(False, eos_token_id=eos)
    got_eos, ahead_eos = run(True, eos_token_id=eos)
    assert got_eos == want_eos and ahead_eos > 0
    first = want_eos[0][0]
    assert first[-1] == eos and len(first) <= 11 and eos not in first[:-1]
