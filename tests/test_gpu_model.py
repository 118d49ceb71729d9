"""The engine against the plain implementation, for every way of cutting the work, in float32 and bfloat16."""

import pytest
import torch

from helpers import (TINY, assert_close, make_engine, mixed_trace, peak_pages, peaky_folder, run_portions,
                     token_ids)
from plain import qwen2_plain as plain
from somi_inference_amd.cache import OutOfPages
from somi_inference_amd.engine import StepEntry, StepError

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]
NAMES = list(TINY)


@pytest.fixture(scope="module")
def peaky_folders(model_folders, tmp_path_factory):
    root = tmp_path_factory.mktemp("peaky")
    return {name: peaky_folder(folder, str(root / name)) for name, folder in model_folders.items()}


@pytest.fixture(scope="module")
def oracle(model_folders, peaky_folders):
    """Plain logits of (folder kind, config name, token tuple), computed once."""
    cache, models = {}, {}

    def get(kind: str, name: str, tokens: list[int]) -> torch.Tensor:
        key = (kind, name, tuple(tokens))
        if key not in cache:
            if (kind, name) not in models:
                models[(kind, name)] = plain.read_model((model_folders if kind == "plain" else peaky_folders)[name])
            cfg, weights = models[(kind, name)]
            cache[key] = plain.model_logits(cfg, weights, tokens)
        return cache[key]
    return get


def folder_of(kind, name, model_folders, peaky_folders):
    return (model_folders if kind == "plain" else peaky_folders)[name]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
@pytest.mark.parametrize("kind", ["plain", "peaky"])
def test_each_request_alone_and_whole(kind, name, dtype, model_folders, peaky_folders, oracle):
    vocab, bs = TINY[name]["config"].vocab_size, TINY[name]["block_size"]
    runner, _ = make_engine(folder_of(kind, name, model_folders, peaky_folders), dtype, bs, 64)
    for length, seed in ((1, 1), (5, 2), (17, 3), (33, 4), (64, 5), (100, 6), (257, 7)):
        tokens = token_ids(vocab, length, seed)
        got = run_portions(runner, f"r{length}", tokens, [length])
        assert_close(got, oracle(kind, name, tokens), dtype, f"{name} {dtype} whole prompt of {length}")
    runner.cache.check_invariants()
    assert runner.cache.free_pages() == [64] * len(runner.cache.groups)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_most_in_one_step_then_the_last_32_one_by_one(name, dtype, peaky_folders, oracle):
    vocab, bs = TINY[name]["config"].vocab_size, TINY[name]["block_size"]
    runner, _ = make_engine(peaky_folders[name], dtype, bs, 32)
    for length in (45, 130):
        tokens = token_ids(vocab, length, 40 + length)
        got = run_portions(runner, "d", tokens, [length - 32] + [1] * 32)
        want = oracle("peaky", name, tokens)
        assert_close(got, want, dtype, f"{name} {dtype} prefill {length - 32} + 32 decoded")
        if dtype == "float32":
            whole = run_portions(runner, "w", tokens, [length])
            assert torch.equal(got, whole), "float32 logits differ between decoding and the whole prompt"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_portions_of_changing_size_down_to_two_tokens(name, dtype, peaky_folders, oracle):
    vocab, bs = TINY[name]["config"].vocab_size, TINY[name]["block_size"]
    runner, _ = make_engine(peaky_folders[name], dtype, bs, 32)
    tokens = token_ids(vocab, 150, 77)
    want = oracle("peaky", name, tokens)
    whole = run_portions(runner, "w", tokens, [150])
    for sizes in ([7, 2, 5, 3, 11, 2, 16, 2, 29], [2], [bs, bs + 1, bs - 1, 2 * bs], [3, 64, 2, 50]):
        got = run_portions(runner, "c", tokens, sizes)
        assert_close(got, want, dtype, f"{name} {dtype} portions {sizes}")
        if dtype == "float32":
            assert torch.equal(got, whole), f"float32 logits depend on the portions {sizes}"
        else:
            assert (got - whole).abs().max() < 2e-2, f"bfloat16 logits depend on the portions {sizes} beyond rounding"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_mixed_batches_with_so_few_pages_that_they_are_used_again(name, dtype, peaky_folders, oracle):
    vocab, bs = TINY[name]["config"].vocab_size, TINY[name]["block_size"]
    lengths = {"a": 70, "b": 45, "c": 100, "d": 33, "e": 64, "f": 90, "g": 2, "h": 51}
    requests = {rid: token_ids(vocab, n, 100 + i) for i, (rid, n) in enumerate(lengths.items())}
    steps = mixed_trace(requests, seed=5)
    pages = peak_pages(steps, bs)
    assert pages < sum((n + bs - 1) // bs for n in lengths.values()), "the trace does not force pages to be used again"
    runner, _ = make_engine(peaky_folders[name], dtype, bs, pages, max_requests=4)
    rows = {rid: [] for rid in requests}
    seen_pages = set()
    reused = False
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
            held = set(p for p in runner.cache.page_list(0, rid) if p >= 0)
            reused = reused or bool(held & seen_pages)
            seen_pages |= held
            runner.end(rid)
        runner.cache.check_invariants()
    assert reused, "no page was used by two requests"
    for rid, tokens in requests.items():
        assert_close(torch.cat(rows[rid]), oracle("peaky", name, tokens), dtype, f"{name} {dtype} mixed request {rid}")
    assert runner.cache.free_pages() == [pages] * len(runner.cache.groups)


@pytest.mark.parametrize("name", ["A", "B"])
def test_float32_engine_on_weights_stored_in_float32(name, tmp_path):
    """The other folders hold bfloat16 values, which a product that rounded its operands to bfloat16 would
    multiply exactly.  Here every tensor is stored in float32 with a full mantissa (and stays so on the device),
    attention is sharpened, and the float32 engine must still meet the float32 tolerance under every cutting."""
    from safetensors.torch import load_file
    from somi_inference_amd.weights import write_random_model
    config, bs = TINY[name]["config"], TINY[name]["block_size"]
    base = write_random_model(str(tmp_path / "f32"), config, seed=TINY[name]["seed"], stored=torch.float32)
    folder = peaky_folder(base, str(tmp_path / "f32_peaky"))
    stored = load_file(f"{folder}/model.safetensors")
    assert all(t.dtype == torch.float32 for t in stored.values())
    some = stored["model.layers.0.mlp.down_proj.weight"]
    assert not torch.equal(some, some.bfloat16().float()), "the stored values would survive a rounding to bfloat16"
    cfg, weights = plain.read_model(folder)
    tokens = token_ids(config.vocab_size, 150, 3)
    want = plain.model_logits(cfg, weights, tokens)
    runner, _ = make_engine(folder, "float32", bs, 32)
    assert runner.model.layers[0].feed_forward.down.weight.dtype == torch.float32
    whole = run_portions(runner, "w", tokens, [150])
    assert_close(whole, want, "float32", f"{name} float32 weights: whole prompt")
    for sizes in ([118] + [1] * 32, [7, 2, 5, 3, 11, 2, 16, 2, 29]):
        got = run_portions(runner, "c", tokens, sizes)
        assert_close(got, want, "float32", f"{name} float32 weights: portions {sizes[:4]}")
        assert torch.equal(got, whole)
    # the bfloat16 engine rounds these weights once, at load: it agrees with the plain implementation run on the
    # rounded values
    lowp, _ = make_engine(folder, "bfloat16", bs, 32)
    rounded = {k: v.bfloat16().float() if v.dim() == 2 else v for k, v in weights.items()}
    assert_close(run_portions(lowp, "w", tokens, [150]), plain.model_logits(cfg, rounded, tokens), "bfloat16",
                 f"{name} float32 weights in the bfloat16 engine")


@pytest.mark.parametrize("dtype", DTYPES)
def test_pages_beyond_two_to_the_31_elements_of_a_cache_tensor(dtype, peaky_folders, oracle):
    """A pool sized for a large GPU: the pool hands out its highest pages first, so the first request's keys
    and values lie past 2^31 elements of their tensors, where a 32-bit offset would wrap."""
    config, bs = TINY["A"]["config"], TINY["A"]["block_size"]
    per_page = config.num_key_value_heads * config.head_dim * bs
    pages = (1 << 31) // per_page + 64
    runner, _ = make_engine(peaky_folders["A"], dtype, bs, pages)
    tokens = token_ids(config.vocab_size, 120, 9)
    got = run_portions(runner, "far", tokens, [70, 9, 9] + [1] * 32)
    assert_close(got, oracle("peaky", "A", tokens), dtype, f"A {dtype} in the highest pages of {pages}")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["B", "C"])
def test_long_decoding_from_a_short_prompt(name, dtype, peaky_folders, oracle):
    vocab, bs = TINY[name]["config"].vocab_size, TINY[name]["block_size"]
    runner, _ = make_engine(peaky_folders[name], dtype, bs, 64)
    tokens = token_ids(vocab, 300, 9)
    got = run_portions(runner, "l", tokens, [3] + [1] * 297)
    assert_close(got, oracle("peaky", name, tokens), dtype, f"{name} {dtype} 297 tokens decoded one by one")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_the_first_tokens_of_a_sequence(name, dtype, model_folders, oracle):
    vocab, bs = TINY[name]["config"].vocab_size, TINY[name]["block_size"]
    runner, _ = make_engine(model_folders[name], dtype, bs, 8)
    tokens = token_ids(vocab, 4, 3)
    want = oracle("plain", name, tokens)
    assert_close(run_portions(runner, "x", tokens[:1], [1]), want[:1], dtype, "a prompt of one token")
    assert_close(run_portions(runner, "y", tokens, [1, 1, 2]), want, dtype, "token by token from the start")
    # only the wanted places come back, in the order asked for
    runner.begin("z")
    got = runner.step([StepEntry("z", tokens, [3, 0])]).cpu()
    runner.end("z")
    assert_close(got, want[[3, 0]], dtype, "wanted places")
    runner.begin("n")
    assert runner.step([StepEntry("n", tokens, [])]).shape == (0, vocab)
    runner.end("n")


def test_step_contract_errors(model_folders):
    runner, config = make_engine(model_folders["A"], "float32", 16, 2)
    with pytest.raises(StepError, match="not live"):
        runner.step([StepEntry("q", [1], [0])])
    runner.begin("q")
    with pytest.raises(StepError, match="outside"):        # out-of-range ids raise, as in the reference
        runner.step([StepEntry("q", [config.vocab_size], [0])])
    with pytest.raises(StepError, match="outside"):
        runner.step([StepEntry("q", [-1], [0])])
    with pytest.raises(StepError, match="wanted place"):
        runner.step([StepEntry("q", [1, 2], [2])])
    with pytest.raises(StepError, match="twice"):
        runner.step([StepEntry("q", [1], [0]), StepEntry("q", [2], [0])])
    with pytest.raises(StepError, match="at least one token"):
        runner.step([StepEntry("q", [], [])])
    before = runner.cache.free_pages()
    with pytest.raises(OutOfPages):
        runner.step([StepEntry("q", [1] * 33, [0])])       # 3 pages, the pool has 2
    assert runner.cache.free_pages() == before and runner.cache.num_tokens("q") == 0
    assert runner.step([StepEntry("q", [1] * 32, [31])]).shape == (1, config.vocab_size)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", NAMES)
def test_decode_steps_of_many_requests_against_the_plain_implementation(name, dtype, peaky_folders, oracle):
    """70, 100, 150 and 260 requests decoding together (the products of 65 to 128 rows in passes and on the 128-row
    tile, beyond on 256-row tiles with K shared by workgroups, logits of many rows in one pass): four steps each,
    through the captured graphs, and after the last one the logits of every request, short and long ones,
    against the plain implementation (a fault may sit in some rows of a tile only: at a pass's edge, in a padded
    row of a graph's bucket)."""
    vocab, bs = TINY[name]["config"].vocab_size, TINY[name]["block_size"]
    pages = 270 * ((40 + 4 + bs - 1) // bs + 1)
    runner, _ = make_engine(peaky_folders[name], dtype, bs, pages, max_requests=270)
    for batch in (70, 100, 150, 260):
        ids = [f"m{batch}_{i}" for i in range(batch)]
        tokens = [token_ids(vocab, 2 + (i * 11) % 39, 500 + batch + i) for i in range(batch)]
        for rid, prompt in zip(ids, tokens):
            runner.begin(rid)
            runner.step([StepEntry(rid, prompt[:-1], [])])
        for step in range(4):
            logits = runner.step([StepEntry(rid, [seq[-1]], [0]) for rid, seq in zip(ids, tokens)])
            if step < 3:
                for seq, token in zip(tokens, logits.argmax(dim=-1).tolist()):
                    seq.append(int(token))
        logits = logits.cpu()
        want = torch.stack([oracle("peaky", name, tokens[i])[-1] for i in range(batch)])
        assert_close(logits, want, dtype, f"{name} {dtype}: {batch} requests after 2 to 44 tokens", per_row=True)
        for rid in ids:
            runner.end(rid)
    runner.cache.check_invariants()
    assert runner.cache.free_pages() == [pages] * len(runner.cache.groups)


@pytest.mark.parametrize("dtype", DTYPES)
def test_captured_decode_steps_replay_like_eager_steps(dtype, model_folders):
    """Decode steps are captured as HIP graphs per number of rows (4, 48 and 80 here, the entries padded up to
    them).  Batches of 3, 40 and 70 requests (the largest takes the products of more than 64 rows inside the
    graph, the others the few-rows kernels that fuse norm, rotation and residual add into the products) are
    replayed several times, with eager work and synchronisations in between, and every replay is compared with
    the same step run without graphs."""
    from somi_inference_amd.models import load_model, make_runner
    from somi_inference_amd.engine import ModelRunner
    from somi_inference_amd.cache import CacheManager
    vocab, bs = TINY["B"]["config"].vocab_size, TINY["B"]["block_size"]
    model, _ = load_model(model_folders["B"], dtype=dtype)
    graphed = make_runner(model, block_size=bs, num_blocks=512, max_requests=80)
    eager_cache = CacheManager(model.cache_needs(), block_size=bs, num_blocks=512, max_requests=80,
                               dtype=model.runtime.dtype, device=model.runtime.device)
    eager = ModelRunner(model, eager_cache, decode_graphs=False)
    assert graphed.decode_graphs and not eager.decode_graphs
    for batch in (3, 40, 70):
        ids = [f"g{batch}_{i}" for i in range(batch)]
        prompts = [token_ids(vocab, 5 + (i * 7) % 23, 300 + i) for i in range(batch)]
        for runner in (graphed, eager):
            for rid, prompt in zip(ids, prompts):
                runner.begin(rid)
                runner.step([StepEntry(rid, prompt, [])])
        last = [p[-1] for p in prompts]
        for step in range(12):
            if batch == 40 and step == 6:
                # five requests end: 35 entries replay the graph of 48 rows that served 40 (rows beyond the entries
                # are padding), no new capture
                captured = len(graphed._graphs)
                for runner in (graphed, eager):
                    for rid in ids[35:]:
                        runner.end(rid)
                ids, last = ids[:35], last[:35]
            entries = [StepEntry(rid, [tok], [0]) for rid, tok in zip(ids, last)]
            want = eager.step(entries).clone()
            got = graphed.step(entries).clone()
            torch.cuda.synchronize()
            if dtype == "float32":
                assert torch.equal(got, want), f"batch {batch}, replay {step}: graph and eager logits differ"
            else:
                # a captured step sizes its key splits for the widest context its block tables allow, an eager
                # step for the actual one: the bfloat16 weights of P.V are rounded relative to another maximum
                assert (got - want).abs().max() < 2e-2, f"batch {batch}, replay {step}"
            last = want.argmax(dim=-1).tolist()
            _ = torch.randn(64, 64, device="cuda:0") @ torch.randn(64, 64, device="cuda:0")   # eager work in between
        if batch == 40:
            assert len(graphed._graphs) == captured, "a batch that shrank within its row bucket was captured again"
        for runner in (graphed, eager):
            for rid in ids:
                runner.end(rid)
    assert graphed.graph_replays >= 36


REAL_SIZES = {
    # one layer of the 7B layer sizes: the shapes the kernels are tuned for
    "7b": dict(hidden_size=3584, intermediate_size=18944, num_hidden_layers=1, num_attention_heads=28,
               num_key_value_heads=4, head_dim=128, rope_theta=1e6, rms_norm_eps=1e-6, tie_word_embeddings=False),
    # two layers of the 0.5B layer sizes: heads of 64, 7 query heads per key/value head, tied embeddings
    "0.5b": dict(hidden_size=896, intermediate_size=4864, num_hidden_layers=2, num_attention_heads=14,
                 num_key_value_heads=2, head_dim=64, rope_theta=1e6, rms_norm_eps=1e-6, tie_word_embeddings=True),
}


@pytest.fixture(scope="module", params=sorted(REAL_SIZES))
def real_size_folder(request, tmp_path_factory):
    """Layers of real layer sizes with a small vocabulary and random weights."""
    from somi_inference_amd.config import Qwen2Config
    from somi_inference_amd.weights import write_random_model
    config = Qwen2Config(vocab_size=1031, **REAL_SIZES[request.param])
    folder = str(tmp_path_factory.mktemp("real") / f"layers_{request.param}")
    write_random_model(folder, config, seed=5)
    return {"float32": peaky_folder(folder, folder + "_peaky", factor=3.0), "bfloat16": folder}, config, request.param


@pytest.mark.parametrize("dtype", DTYPES)
def test_layers_of_real_sizes_under_all_cuttings(dtype, real_size_folder):
    """With sums over up to 18,944 terms the order of float32 additions shows: the float32 engine is held to
    the accuracy of the plain float32 implementation itself, both measured against the plain implementation
    in float64 (its error may be a few times the plain one's, not more).  The float32 run uses sharpened
    attention (single keys decide); in bfloat16 that sharpening amplifies the rounding of q and k into
    per-cent changes of the weights, so the bfloat16 run uses the weights as drawn."""
    folders, config, sizes = real_size_folder
    folder = folders[dtype]
    cfg, weights = plain.read_model(folder)
    tokens = token_ids(config.vocab_size, 333, 8)
    want = plain.model_logits(cfg, weights, tokens)
    cfg64, weights64 = plain.read_model(folder, dtype=torch.float64)
    want64 = plain.model_logits(cfg64, weights64, tokens)
    plain_error = float((want.double() - want64).abs().max())

    def check(got, rows, what):
        if dtype == "float32":
            error = float((got.double().cpu() - want64[rows]).abs().max())
            assert error <= 4 * plain_error + 1e-6, f"{what}: error {error:.3e}, the plain float32 implementation's {plain_error:.3e}"
        else:
            # bfloat16 rounds to 2^-9 relative at about six places per layer (normed input, projections, gate,
            # attention weights, sub-layer outputs); independent roundings add up to roughly half a per cent of
            # the logits' size.  The bounds sit at four times that (rms) and at 3 % for a single element; a
            # fault (wrong key, page or row) changes logits by their own size.
            ref = want[rows]
            error = (got.float().cpu() - ref).abs()
            assert float(error.max()) <= 0.03 * float(ref.abs().max()), f"{what}: max error {float(error.max()):.3e}"
            assert float(error.pow(2).mean().sqrt()) <= 0.02 * float(ref.pow(2).mean().sqrt()), \
                f"{what}: rms error {float(error.pow(2).mean().sqrt()):.3e} of rms {float(ref.pow(2).mean().sqrt()):.3e}"

    runner, _ = make_engine(folder, dtype, 16, 64, max_requests=4)
    everything = list(range(len(tokens)))
    whole = run_portions(runner, "w", tokens, [333])
    check(whole, everything, f"{sizes} layer sizes {dtype}: whole prompt")
    cut = run_portions(runner, "c", tokens, [150, 2, 37, 1, 1, 64, 9, 33] + [1] * 36)
    check(cut, everything, f"{sizes} layer sizes {dtype}: portions and decoded tokens")
    if dtype == "float32":
        assert torch.equal(cut, whole)
    # three requests decoding together after prompts of different lengths
    prompts = {"a": tokens[:40], "b": tokens[:111], "c": tokens[:290]}
    for rid, prompt in prompts.items():
        runner.begin(rid)
        runner.step([StepEntry(rid, prompt, [])])
    for step in range(20):
        entries = [StepEntry(rid, [tokens[len(p) + step]], [0]) for rid, p in prompts.items()]
        got = runner.step(entries).cpu()
        check(got, [len(p) + step for p in prompts.values()], f"{sizes} layer sizes {dtype}: batched decode step {step}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_decoding_from_tokens_that_are_still_on_the_device(dtype, model_folders):
    """A decode step may take its tokens from the sampler's device tensor before the host has read them (the
    host then works one step ahead of the device): the same tokens come out as when every step waits."""
    from somi_inference_amd.sampling import Sampler, SamplingParams
    name = "B"
    vocab = TINY[name]["config"].vocab_size
    prompts = {"a": token_ids(vocab, 21, 1), "b": token_ids(vocab, 9, 2), "c": token_ids(vocab, 40, 3)}
    sampler, greedy = Sampler(), SamplingParams(temperature=0.0)

    def start(engine):
        first = []
        for rid, prompt in prompts.items():
            engine.begin(rid)
            first.append(sampler.sample(engine.step([StepEntry(rid, prompt, [len(prompt) - 1])]), greedy)[0])
        return first

    waiting, _ = make_engine(model_folders[name], dtype, block_size=8, num_blocks=40)
    tokens, want = start(waiting), []
    for _ in range(20):
        tokens = sampler.sample(waiting.step([StepEntry(rid, [t], [0]) for rid, t in zip(prompts, tokens)]), greedy)
        want.append(tokens)

    ahead, _ = make_engine(model_folders[name], dtype, block_size=8, num_blocks=40)
    tokens, got = start(ahead), []
    placeholders = [StepEntry(rid, [0], [0]) for rid in prompts]
    newest = sampler.sample_async(ahead.step([StepEntry(rid, [t], [0]) for rid, t in zip(prompts, tokens)]), greedy)
    for _ in range(19):
        older, newest = newest, sampler.sample_async(ahead.step(placeholders, device_tokens=newest.device), greedy)
        got.append(older.tolist())
    got.append(newest.tolist())
    assert got == want
    assert ahead.graph_replays > 0
    with pytest.raises(StepError, match="one token each"):
        ahead.step([StepEntry("a", [1, 2], [1])], device_tokens=newest.device[:1])
    with pytest.raises(StepError, match="int32"):
        ahead.step(placeholders, device_tokens=newest.device[:2])
