"""Each part alone against the plain implementation, at sizes of its own, and parts chosen layer by layer."""

import pytest
import torch

from plain import qwen2_plain as plain
from somi_inference_amd.cache import CacheManager
from somi_inference_amd.engine import StepEntry, build_step
from somi_inference_amd.models import DecoderModel, LayerSpec, ModelPlan
from somi_inference_amd.parts import (GroupedQueryAttention, LMHead, PartSpec, PreNormBlock, ResidualStream, RMSNorm,
                                      RotaryPosition, Runtime, SwiGLU, TokenEmbedding)
from somi_inference_amd.weights import RandomSource

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
SPLITS = (GroupedQueryAttention.entry_split,)      # what the runner takes from the model's mixers and hands to build_step
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": dict(atol=2e-5, rtol=1e-4), "bfloat16": dict(atol=3e-2, rtol=3e-2)}


@pytest.fixture(autouse=True)
def seeded():
    torch.manual_seed(1234)
    torch.cuda.manual_seed(1234)


def close(got, want, dtype):
    """Rounding errors scale with the size of the activations: bound them against the largest element
    (2^-8 per bfloat16 rounding, a handful of roundings per part)."""
    scale = float(want.abs().max())
    rel = 2e-5 if dtype == "float32" else 2e-2
    torch.testing.assert_close(got.float().cpu(), want, atol=rel * max(scale, 1e-3), rtol=rel)


def rows(out):
    """A part's output as a tensor: its last projection may come back not yet computed."""
    return out.materialize() if hasattr(out, "materialize") else out


def load_random(part, dtype, seed=0, scale=None):
    """Load a part from seeded random tensors; returns them as float32 CPU tensors for the plain side."""
    source = RandomSource(part.weight_specs(), seed)
    kept = {}

    def fetch(name):
        spec = next(s for s in part.weight_specs() if s.name == name)
        tensor = source.read(name, DEV)
        if scale and spec.role == "matrix":
            tensor = (tensor.float() * scale).to(tensor.dtype)
        kept[name] = tensor.float().cpu()
        return tensor.to(DT[dtype] if spec.role == "matrix" else torch.float32).contiguous()
    part.load(fetch, Runtime(DT[dtype], DEV))
    return kept


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_rmsnorm_part_and_residual_stream(dtype):
    norm = RMSNorm("n", hidden_size=136, eps=2e-5)
    w = load_random(norm, dtype)
    h = torch.randn(6, 136, device=DEV)
    torch.testing.assert_close(norm.forward(h.clone()).float().cpu(), plain.rms_norm(h.cpu(), w["n.weight"], 2e-5), **TOL[dtype])
    stream = ResidualStream(h.clone())
    d1 = torch.randn(6, 136, device=DEV).to(DT[dtype])
    d2 = torch.randn(6, 136, device=DEV).to(DT[dtype])
    stream.add(d1)
    x = stream.normed(norm)                              # the fused add + norm
    torch.testing.assert_close(x.float().cpu(), plain.rms_norm((h + d1.float()).cpu(), w["n.weight"], 2e-5), **TOL[dtype])
    stream.add(d2)
    torch.testing.assert_close(stream.settle(), h + d1.float() + d2.float(), atol=1e-6, rtol=1e-6)
    assert stream.h.dtype == torch.float32               # the residual sum is 32-bit in both engines


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_swiglu_part(dtype):
    ffn = SwiGLU("m", hidden_size=72, intermediate_size=200)
    w = load_random(ffn, dtype, scale=5.0)
    assert tuple(ffn.gate_up.weight.shape) == (400, 72)              # merged weight (2I, H): reference test_qwen2_mlp.py:17-20
    x = torch.randn(9, 72, device=DEV).to(DT[dtype])
    want = plain.swiglu(x.float().cpu(), w["m.gate_proj.weight"], w["m.up_proj.weight"], w["m.down_proj.weight"])
    close(rows(ffn.forward(x)), want, dtype)


def attention_setup(dtype, nq, nkv, d, hidden, window=None, theta=1e4, block_size=4, seed=0):
    attn = GroupedQueryAttention("a", hidden_size=hidden, num_heads=nq, num_kv_heads=nkv, head_dim=d,
                                 position=PartSpec("rotary", {"head_dim": d, "theta": theta}), window=window)
    w = load_random(attn, dtype, seed=seed, scale=8.0)
    cache = CacheManager([attn.cache_spec()], block_size=block_size, num_blocks=64, max_requests=4,
                         dtype=DT[dtype], device=DEV)
    cfg = dict(num_attention_heads=nq, num_key_value_heads=nkv, head_dim=d, rope_theta=theta)
    return attn, w, cache, cfg


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nq, nkv, d, hidden, window", [(12, 2, 16, 40, None), (8, 1, 32, 72, None), (6, 6, 48, 56, 9)])
def test_attention_part_whole_and_in_portions(dtype, nq, nkv, d, hidden, window):
    attn, w, cache, cfg = attention_setup(dtype, nq, nkv, d, hidden, window)
    x = torch.randn(37, hidden, device=DEV).to(DT[dtype])
    want = plain.attention_block(x.float().cpu(), w, "a", cfg, torch.arange(37), window)
    for sizes in ([37], [5, 2, 9, 1, 1, 19]):
        cache.register("r")
        outs, at = [], 0
        for size in sizes:
            cache.reserve("r", size)
            step = build_step([StepEntry("r", [0] * size, [])], cache, DEV, SPLITS)
            outs.append(rows(attn.forward(x[at:at + size].contiguous(), step, cache.layer_caches[0])))
            cache.commit("r", size)
            at += size
        cache.free("r")
        close(torch.cat(outs), want, dtype)


@pytest.mark.parametrize("n_rows", [40, 64, 65, 81, 100, 128, 129])
def test_attention_part_reads_rows_still_to_be_normed(n_rows):
    """bfloat16 rows as a product into the residual stream leaves them (weighted, with their sums of squares): up to 64
    the q/k/v product norms, rotates and stores them in one kernel, up to 128 in passes of 64 that cut through a
    request, beyond by the many-rows kernels.  Three requests' prompts in one step."""
    from somi_inference_amd.parts.linear import NormedRows
    nq, nkv, d, hidden = 8, 2, 32, 72
    attn, w, cache, cfg = attention_setup("bfloat16", nq, nkv, d, hidden, block_size=8)
    ffn = SwiGLU("m", hidden_size=hidden, intermediate_size=96)
    wf = load_random(ffn, "bfloat16", scale=4.0)
    norm = RMSNorm("n", hidden_size=hidden, eps=1e-5)
    wn = load_random(norm, "bfloat16")
    h0 = torch.randn(n_rows, hidden, device=DEV)
    x0 = norm.forward(h0)
    stream = ResidualStream(h0.clone())
    stream.add(ffn.forward(x0))
    lazy = stream.normed(norm, lazy=True)
    assert isinstance(lazy, NormedRows)
    sizes = [n_rows // 2, n_rows // 3, n_rows - n_rows // 2 - n_rows // 3]
    for i, size in enumerate(sizes):
        cache.register(i)
        cache.reserve(i, size)
    step = build_step([StepEntry(i, [0] * size, []) for i, size in enumerate(sizes)], cache, DEV, SPLITS)
    got = rows(attn.forward(lazy, step, cache.layer_caches[0]))
    h1 = h0.cpu() + plain.swiglu(x0.float().cpu(), wf["m.gate_proj.weight"], wf["m.up_proj.weight"], wf["m.down_proj.weight"])
    x1 = plain.rms_norm(h1, wn["n.weight"], 1e-5)
    at = 0
    for size in sizes:
        want = plain.attention_block(x1[at:at + size], w, "a", cfg, torch.arange(size), None)
        close(got[at:at + size], want, "bfloat16")
        at += size


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_attention_part_far_key_among_hundreds_and_window_edge(dtype):
    """One query and one far key are made to agree strongly, so that key alone decides the output:
    reading the wrong page or slot, or a window edge off by one, changes the result visibly."""
    nq, nkv, d, hidden, length = 4, 2, 16, 16, 300
    for window, far in ((None, 3), (64, length - 64), (64, length - 65)):
        attn, w, cache, cfg = attention_setup(dtype, nq, nkv, d, hidden, window, theta=1e4, block_size=16, seed=4)
        # pick (deterministically) inputs for which the far key decides the last token's output whenever it
        # is visible: a loud key, a query that matches it, and a sign of their product that favours it
        for attempt in range(50):
            gen = torch.Generator().manual_seed(100 + attempt)
            x = torch.randn(length, hidden, generator=gen) * 0.1
            x[far] *= 60.0
            x[length - 1] = x[far]
            want = plain.attention_block(x, w, "a", cfg, torch.arange(length), None)
            muted = x.clone()
            muted[far] = 0.0
            if (plain.attention_block(muted, w, "a", cfg, torch.arange(length), None)[-1] - want[-1]).abs().max() > 0.1:
                break
        else:
            raise AssertionError("no input found in which the far key matters")
        x = x.to(DEV).to(DT[dtype])
        want = plain.attention_block(x.float().cpu(), w, "a", cfg, torch.arange(length), window)
        cache.register("r")
        cache.reserve("r", length - 1)
        attn.forward(x[:length - 1].contiguous(), build_step([StepEntry("r", [0] * (length - 1), [])], cache, DEV, SPLITS),
                     cache.layer_caches[0])
        cache.commit("r", length - 1)
        cache.reserve("r", 1)
        got = rows(attn.forward(x[length - 1:].contiguous(), build_step([StepEntry("r", [0], [])], cache, DEV, SPLITS),
                                cache.layer_caches[0]))
        if dtype == "float32":
            torch.testing.assert_close(got.cpu(), want[-1:], atol=1e-4, rtol=1e-3)
        else:
            close(got, want[-1:], dtype)
        # the far key matters exactly when it is inside the window
        x2 = x.float().cpu()
        x2[far] = 0.0
        moved = (plain.attention_block(x2, w, "a", cfg, torch.arange(length), window)[-1] - want[-1]).abs().max()
        inside = window is None or far > length - 1 - window
        assert (moved > 1e-2) == inside, f"window {window}, far key {far}: moved {moved}"


def test_attention_part_rejects_indivisible_heads():
    with pytest.raises(ValueError, match="divisible"):       # reference: models/qwen2.py:116-123
        GroupedQueryAttention("a", hidden_size=8, num_heads=5, num_kv_heads=2, head_dim=4,
                              position=PartSpec("none", {}))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_embedding_and_head_tied_or_not(dtype):
    emb = TokenEmbedding("e", vocab_size=97, hidden_size=24)
    w = load_random(emb, dtype, scale=20.0)
    ids = torch.tensor([0, 96, 5, 5], dtype=torch.int32, device=DEV)
    assert torch.equal(emb.forward(ids).cpu(), w["e.weight"][ids.long().cpu()])
    x = torch.randn(3, 24, device=DEV).to(DT[dtype])
    tied = LMHead("h", vocab_size=97, hidden_size=24, tied=True)
    assert tied.weight_specs() == []
    tied.load(lambda name: None, Runtime(DT[dtype], DEV))
    tied.tie(emb)
    logits = tied.forward(x)
    assert logits.dtype == torch.float32                     # logits are float32 in both engines
    torch.testing.assert_close(logits.cpu(), x.float().cpu() @ w["e.weight"].t(), **TOL[dtype])   # reference qwen2_adapter.py:60-62
    own = LMHead("h", vocab_size=97, hidden_size=24)
    wh = load_random(own, dtype, seed=9, scale=20.0)
    torch.testing.assert_close(own.forward(x).cpu(), x.float().cpu() @ wh["h.weight"].t(), **TOL[dtype])


def test_block_with_zero_projections_is_the_identity():
    # reference: tests/models/test_qwen2_decoder_layer.py:31-62
    norm = PartSpec("rmsnorm", {"hidden_size": 32, "eps": 1e-6})
    block = PreNormBlock("l", mixer=PartSpec("gqa_attention", {"hidden_size": 32, "num_heads": 4, "num_kv_heads": 2,
                                                               "head_dim": 8, "position": PartSpec("rotary", {"head_dim": 8, "theta": 1e4})}),
                         feed_forward=PartSpec("swiglu", {"hidden_size": 32, "intermediate_size": 48}),
                         mixer_norm=norm, ffn_norm=norm)
    block.load(lambda name: (torch.ones if "norm" in name else torch.zeros)(
        next(s.shape for s in block.weight_specs() if s.name == name), device=DEV), Runtime(torch.float32, DEV))
    cache = CacheManager([block.mixer.cache_spec()], block_size=4, num_blocks=8, max_requests=2,
                         dtype=torch.float32, device=DEV)
    cache.register("r")
    cache.reserve("r", 5)
    h = torch.randn(5, 32, device=DEV)
    stream = ResidualStream(h.clone())
    block.forward(stream, build_step([StepEntry("r", [0] * 5, [])], cache, DEV, SPLITS), cache.layer_caches[0])
    assert torch.equal(stream.settle(), h)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_plan_may_choose_parts_layer_by_layer_and_run_a_layer_twice(dtype):
    """Layers with different mixers (full, windowed, another head count) and feed-forward widths in one
    model; the run order names layer 1 twice; each run has a cache of its own."""
    hidden, vocab = 48, 61

    def layer(index, nq, nkv, d, window, inter):
        norm = PartSpec("rmsnorm", {"hidden_size": hidden, "eps": 1e-6})
        mixer = PartSpec("gqa_attention", {"hidden_size": hidden, "num_heads": nq, "num_kv_heads": nkv, "head_dim": d,
                                           "position": PartSpec("rotary", {"head_dim": d, "theta": 1e4}), "window": window})
        ffn = PartSpec("swiglu", {"hidden_size": hidden, "intermediate_size": inter})
        return LayerSpec(f"model.layers.{index}", PartSpec("pre_norm", {"mixer": mixer, "feed_forward": ffn,
                                                                         "mixer_norm": norm, "ffn_norm": norm}))
    shapes = [(4, 2, 16, None, 64), (6, 1, 8, 7, 100), (2, 2, 32, None, 36)]
    plan = ModelPlan(
        embedding=PartSpec("token_embedding", {"vocab_size": vocab, "hidden_size": hidden}), embedding_prefix="model.embed_tokens",
        layers=tuple(layer(i, *s) for i, s in enumerate(shapes)), order=(0, 1, 1, 2),
        final_norm=PartSpec("rmsnorm", {"hidden_size": hidden, "eps": 1e-6}), final_norm_prefix="model.norm",
        head=PartSpec("lm_head", {"vocab_size": vocab, "hidden_size": hidden, "tied": True}), head_prefix="lm_head",
        vocab_size=vocab)
    model = DecoderModel(plan, Runtime(DT[dtype], DEV))
    kept = {}
    source = RandomSource(model.weight_specs(), 3)

    class Keeping(RandomSource):
        def read(self, name, device):
            tensor = super().read(name, device)
            if "_proj.weight" in name:
                tensor = (tensor.float() * 6.0).to(tensor.dtype)
            kept[name] = tensor.float().cpu()
            return tensor
    model.load(Keeping(model.weight_specs(), 3))
    needs = model.cache_needs()
    assert len(needs) == 4 and needs[1] == needs[2] and needs[1].window == 7
    cache = CacheManager(needs, block_size=8, num_blocks=16, max_requests=2, dtype=DT[dtype], device=DEV)
    assert len(cache.groups) == 2 and cache.layer_caches[1].k is not cache.layer_caches[2].k
    tokens = torch.randint(0, vocab, (29,), generator=torch.Generator().manual_seed(1)).tolist()

    # the plain side: the same layers in the same order
    h = kept["model.embed_tokens.weight"][torch.tensor(tokens)]
    for index in plan.order:
        nq, nkv, d, window, _ = shapes[index]
        cfg = dict(num_attention_heads=nq, num_key_value_heads=nkv, head_dim=d, rope_theta=1e4)
        p = f"model.layers.{index}"
        h = h + plain.attention_block(plain.rms_norm(h, kept[f"{p}.input_layernorm.weight"], 1e-6), kept,
                                      f"{p}.self_attn", cfg, torch.arange(29), window)
        h = h + plain.swiglu(plain.rms_norm(h, kept[f"{p}.post_attention_layernorm.weight"], 1e-6),
                             kept[f"{p}.mlp.gate_proj.weight"], kept[f"{p}.mlp.up_proj.weight"], kept[f"{p}.mlp.down_proj.weight"])
    want = plain.rms_norm(h, kept["model.norm.weight"], 1e-6) @ kept["model.embed_tokens.weight"].t()

    from somi_inference_amd.engine import ModelRunner
    runner = ModelRunner(model, cache)
    for sizes in ([29], [3, 11, 2, 13]):
        runner.begin("r")
        outs, at = [], 0
        for size in sizes:
            outs.append(runner.step([StepEntry("r", tokens[at:at + size], list(range(size)))]))
            at += size
        runner.end("r")
        torch.testing.assert_close(torch.cat(outs).cpu(), want, **TOL[dtype])


def test_rotary_part_offers_the_reference_table():
    rope = RotaryPosition("p", head_dim=8, theta=1_000_000.0)
    rope.load(lambda name: None, Runtime(torch.float32, DEV))
    inv_freq, rotary_dim = rope.rotation_table()
    assert rotary_dim == 8 and inv_freq.dtype == torch.float32
    # reference: cos_cached[1][1] = cos(1e6^-0.25) for dim 8 (tests/models/test_qwen2.py:75-88)
    assert inv_freq.cpu().tolist() == pytest.approx([1.0, 1e6 ** -0.25, 1e6 ** -0.5, 1e6 ** -0.75], rel=1e-6)


@pytest.mark.parametrize("n_rows", [7, 40, 64, 65, 100, 128, 129, 300])
def test_bfloat16_rows_take_the_add_and_the_norm_inside_the_products(n_rows):
    """Steps in bfloat16, of a few rows (the decode kernels) and of many (the many-rows kernel): a block's last projections arrive at the residual stream uncomputed and are
    added to it by the kernel that computes them; the next norm is applied by the projection that reads the
    rows.  The stream ends up where separate add and norm kernels put it (up to the rounding of the deltas to
    bfloat16, which the fused way skips)."""
    from somi_inference_amd.parts.linear import DeferredProduct, NormedRows
    hidden, inter = 96, 160
    ffn = SwiGLU("m", hidden_size=hidden, intermediate_size=inter)
    w = load_random(ffn, "bfloat16", scale=4.0)
    norm = RMSNorm("n", hidden_size=hidden, eps=1e-5)
    wn = load_random(norm, "bfloat16")
    h0 = torch.randn(n_rows, hidden, device=DEV)
    x = norm.forward(h0)
    out = ffn.forward(x)
    assert isinstance(out, DeferredProduct) and out.shape == (n_rows, hidden)
    # the fused way through the stream
    stream = ResidualStream(h0.clone())
    stream.add(out)
    lazy = stream.normed(norm, lazy=True)
    assert isinstance(lazy, NormedRows)
    lazy_rows = lazy.materialize().float()                       # before the stream moves on
    assert torch.equal(lazy.weighted, (norm.weight * stream.h).to(torch.bfloat16))
    second = ffn.forward(lazy)                                   # norm + gate_up + SiLU.up in one kernel
    assert isinstance(second, DeferredProduct)
    stream.add(second)
    fused = stream.settle().clone()
    # the separate way
    plain_stream = ResidualStream(h0.clone())
    plain_stream.add(out.materialize())
    x2 = plain_stream.normed(norm)
    assert torch.is_tensor(x2)
    torch.testing.assert_close(lazy_rows, x2.float(), atol=2e-2, rtol=2e-2)
    plain_stream.add(rows(ffn.forward(x2)))
    separate = plain_stream.settle()
    scale = float(separate.abs().max())
    torch.testing.assert_close(fused, separate, atol=scale * 2 ** -6, rtol=2 ** -6)
    # against float32 formulas
    h1 = h0.cpu() + plain.swiglu(x.float().cpu(), w["m.gate_proj.weight"], w["m.up_proj.weight"], w["m.down_proj.weight"])
    x2_plain = plain.rms_norm(h1, wn["n.weight"], 1e-5)
    h2 = h1 + plain.swiglu(x2_plain, w["m.gate_proj.weight"], w["m.up_proj.weight"], w["m.down_proj.weight"])
    close(fused, h2, "bfloat16")
    # float32 stays with the separate kernels
    ffn32 = SwiGLU("m", hidden_size=hidden, intermediate_size=inter)
    load_random(ffn32, "float32")
    assert torch.is_tensor(ffn32.forward(torch.randn(7, hidden, device=DEV)))
