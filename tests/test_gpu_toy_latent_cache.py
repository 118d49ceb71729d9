"""A toy mixer that keeps ONE tensor per token (a latent vector, in float32, in pages of its own size) is
defined here, registered, built and stepped through the engine's own runner and cache manager beside an
ordinary attention layer whose checkpoint stores q/k/v and gate/up as single matrices under other names,
without a change to the package's files.  The model is compared with a plain computation written here for
every way of cutting the work: whole, most of it at once and the last tokens one by one, portions of
changing size, and mixed with other requests in a pool so small that pages are used again."""

import pytest
import torch

from helpers import mixed_trace, peak_pages, token_ids
from plain import qwen2_plain as plain
from somi_inference_amd.cache import CacheManager
from somi_inference_amd.engine import ModelRunner, StepEntry
from somi_inference_amd.models import DecoderModel, LayerSpec, ModelPlan
from somi_inference_amd.parts import (PAGE, Mixer, PagedSpec, PageTensor, PartSpec, Runtime, register_part,
                                      unregister_part)
from somi_inference_amd.weights import MATRIX, Init, RandomSource, WeightSpec

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": dict(atol=3e-5, rtol=1e-4), "bfloat16": dict(atol=4e-2, rtol=4e-2)}
HIDDEN, VOCAB, EPS, LATENT = 40, 53, 1e-5, 12
LATENT_PAGE, ENGINE_PAGE = 3, 8
WINDOW = 7


class LatentMixer(Mixer):
    """c[t] = D x[t] is all that is kept of a token; token t reads the latents of the tokens before it (those of
    the window, if there is one) with weights softmax(q[t] . c[s] / sqrt(L)), q[t] = Q x[t], and puts out
    O sum_s p[s] c[s]."""

    def __init__(self, prefix, hidden_size, latent, window=None):
        super().__init__(prefix)
        self.hidden_size, self.latent, self.window = hidden_size, latent, window

    def weight_specs(self):
        return [WeightSpec(self.name("down.weight"), (self.latent, self.hidden_size), MATRIX, Init(0.0, 0.3)),
                WeightSpec(self.name("query.weight"), (self.latent, self.hidden_size), MATRIX, Init(0.0, 0.3)),
                WeightSpec(self.name("out.weight"), (self.hidden_size, self.latent), MATRIX, Init(0.0, 0.2))]

    def load(self, fetch, runtime):
        super().load(fetch, runtime)
        self.down, self.query, self.out = (fetch(self.name(f"{n}.weight")).float() for n in ("down", "query", "out"))

    def cache_spec(self):
        return PagedSpec((PageTensor("latent", (PAGE, self.latent), torch.float32),), self.window, LATENT_PAGE)

    def forward(self, x, step, cache):
        view, kept = step.paged[cache.group], cache.tensors["latent"]
        assert view.page_size == cache.page_size == LATENT_PAGE and kept.dtype == torch.float32
        x32 = x.float()
        kept.view(-1, self.latent)[view.slot_mapping.long()] = x32 @ self.down.t()
        queries = x32 @ self.query.t()
        out = torch.empty_like(x32)
        for e, entry in enumerate(step.entries):
            context = entry.first_position + entry.length
            pages = view.block_table[e, :(context + LATENT_PAGE - 1) // LATENT_PAGE].long()
            latents = kept[pages].reshape(-1, self.latent)[:context]      # pages a window has passed read page 0
            for t in range(entry.length):
                at = entry.first_position + t
                seen = latents[max(0, at - self.window + 1) if self.window else 0:at + 1]
                weights = torch.softmax(seen @ queries[entry.start + t] * self.latent ** -0.5, dim=0)
                out[entry.start + t] = self.out @ (weights @ seen)
        return out.to(x.dtype)


def plain_latent(x, w, prefix, window):
    c, q = x @ w[f"{prefix}.down.weight"].t(), x @ w[f"{prefix}.query.weight"].t()
    scores = q @ c.t() * LATENT ** -0.5
    t = x.shape[0]
    rows, cols = torch.arange(t)[:, None], torch.arange(t)[None, :]
    hidden = cols > rows
    if window:
        hidden = hidden | (cols < rows - window + 1)
    weights = torch.softmax(scores.masked_fill(hidden, float("-inf")), dim=-1)
    return weights @ c @ w[f"{prefix}.out.weight"].t()


@pytest.fixture
def latent_registered():
    register_part("mixer", "toy_latent", LatentMixer)
    yield
    unregister_part("mixer", "toy_latent")


NORM = PartSpec("rmsnorm", {"hidden_size": HIDDEN, "eps": EPS})


def the_plan():
    latent = lambda window: PartSpec("toy_latent", {"hidden_size": HIDDEN, "latent": LATENT, "window": window})
    attention = PartSpec("gqa_attention", {
        "hidden_size": HIDDEN, "num_heads": 4, "num_kv_heads": 2, "head_dim": 16,
        "position": PartSpec("rotary", {"head_dim": 16, "theta": 1e4}),
        "names": {"qkv": "wqkv", "o": "wo"}})
    ffn = PartSpec("swiglu", {"hidden_size": HIDDEN, "intermediate_size": 72})
    ffn_fused = PartSpec("swiglu", {"hidden_size": HIDDEN, "intermediate_size": 72,
                                    "names": {"gate_up": "w13", "down": "w2"}})
    mixers = [latent(None), attention, latent(WINDOW), latent(None)]
    layers = tuple(LayerSpec(f"model.layers.{i}", PartSpec("pre_norm", {
        "mixer": mixer, "feed_forward": ffn_fused if i == 1 else ffn, "mixer_norm": NORM, "ffn_norm": NORM}))
        for i, mixer in enumerate(mixers))
    return ModelPlan(embedding=PartSpec("token_embedding", {"vocab_size": VOCAB, "hidden_size": HIDDEN}),
                     embedding_prefix="model.embed_tokens", layers=layers, final_norm=NORM,
                     final_norm_prefix="model.norm",
                     head=PartSpec("lm_head", {"vocab_size": VOCAB, "hidden_size": HIDDEN, "tied": True}),
                     head_prefix="lm_head", vocab_size=VOCAB)


def build(dtype, num_blocks, max_requests=4, seed=9):
    model = DecoderModel(the_plan(), Runtime(DT[dtype], DEV))
    kept = {}

    class Keeping(RandomSource):
        def read(self, name, device):
            tensor = super().read(name, device)
            if "wqkv.weight" in name:
                tensor = (tensor.float() * 5.0).to(tensor.dtype)
            kept[name] = tensor.float().cpu()
            return tensor
    model.load(Keeping(model.weight_specs(), seed))
    cache = CacheManager(model.cache_needs(), block_size=ENGINE_PAGE, num_blocks=num_blocks, max_requests=max_requests,
                         dtype=DT[dtype], device=DEV)
    return ModelRunner(model, cache), kept


def plain_logits(tokens, w):
    """The toy model on a whole sequence, without a cache."""
    t = len(tokens)
    positions = torch.arange(t)
    h = w["model.embed_tokens.weight"][tokens]
    for i, window in enumerate([None, "attention", WINDOW, None]):
        prefix = f"model.layers.{i}"
        x = plain.rms_norm(h, w[f"{prefix}.input_layernorm.weight"], EPS)
        if window == "attention":
            qkv = plain.linear(x, w[f"{prefix}.self_attn.wqkv.weight"], w[f"{prefix}.self_attn.wqkv.bias"])
            q, k, v = qkv.split([64, 32, 32], dim=-1)
            cos, sin = plain.rope_cos_sin(positions, 16, 1e4)
            q = plain.apply_rope(q.view(t, 4, 16).transpose(0, 1), cos, sin)
            k = plain.apply_rope(k.view(t, 2, 16).transpose(0, 1), cos, sin)
            attended = plain.causal_attention(q, k, v.view(t, 2, 16).transpose(0, 1))
            h = h + plain.linear(attended.transpose(0, 1).reshape(t, 64), w[f"{prefix}.self_attn.wo.weight"])
        else:
            h = h + plain_latent(x, w, f"{prefix}.self_attn", window)
        x = plain.rms_norm(h, w[f"{prefix}.post_attention_layernorm.weight"], EPS)
        if i == 1:
            gate, up = w[f"{prefix}.mlp.w13.weight"].chunk(2, dim=0)
            h = h + plain.swiglu(x, gate, up, w[f"{prefix}.mlp.w2.weight"])
        else:
            h = h + plain.swiglu(x, w[f"{prefix}.mlp.gate_proj.weight"], w[f"{prefix}.mlp.up_proj.weight"],
                                 w[f"{prefix}.mlp.down_proj.weight"])
    return plain.rms_norm(h, w["model.norm.weight"], EPS) @ w["model.embed_tokens.weight"].t()


def feed(runner, rid, tokens, sizes):
    runner.begin(rid)
    outs, at = [], 0
    for size in sizes:
        outs.append(runner.step([StepEntry(rid, tokens[at:at + size], list(range(size)))]).cpu())
        at += size
    assert at == len(tokens)
    runner.end(rid)
    return torch.cat(outs)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_groups_by_what_they_store_and_the_four_cuttings(latent_registered, dtype):
    runner, w = build(dtype, num_blocks=12)
    cache = runner.cache
    # full latents, keys and values, windowed latents: three groups, each with pages of its own size over
    # the same 96 tokens; the two full latent layers share tables and have tensors of their own
    assert [(g.window, g.page_size, g.pool.num_pages, g.runs) for g in cache.groups] == [
        (None, LATENT_PAGE, 32, [0, 3]), (None, ENGINE_PAGE, 12, [1]), (WINDOW, LATENT_PAGE, 32, [2])]
    assert cache.layer_caches[0].tensors["latent"].shape == (32, LATENT_PAGE, LATENT)
    assert cache.layer_caches[0].tensors["latent"].dtype == torch.float32
    assert cache.layer_caches[1].k.shape == (12, 2, ENGINE_PAGE, 16) and cache.layer_caches[1].k.dtype == DT[dtype]
    names = {spec.name for spec in runner.model.weight_specs()}
    assert {"model.layers.1.self_attn.wqkv.weight", "model.layers.1.self_attn.wqkv.bias", "model.layers.1.self_attn.wo.weight",
            "model.layers.1.mlp.w13.weight", "model.layers.1.mlp.w2.weight"} <= names
    assert not any("q_proj" in n or "layers.1.mlp.gate_proj" in n for n in names)

    tokens = token_ids(VOCAB, 75, seed=3)
    want = plain_logits(tokens, w)
    cuttings = {"whole": [75], "most and the last 32 one by one": [43] + [1] * 32,
                "portions of changing size": [5, 2, 13, 3, 2, 17, 7, 2, 9, 15]}
    for what, sizes in cuttings.items():
        got = feed(runner, what, tokens, sizes)
        torch.testing.assert_close(got, want, **TOL[dtype], msg=lambda m: f"{dtype} {what}: {m}")
        cache.check_invariants()
    assert cache.free_pages() == [32, 12, 32]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_mixed_requests_reuse_pages_of_every_group(latent_registered, dtype):
    lengths = {"a": 40, "b": 23, "c": 57, "d": 2, "e": 31, "f": 48}
    requests = {rid: token_ids(VOCAB, n, 40 + i) for i, (rid, n) in enumerate(lengths.items())}
    steps = mixed_trace(requests, seed=11, max_live=3)
    pages = peak_pages(steps, ENGINE_PAGE)
    assert pages < sum((n + ENGINE_PAGE - 1) // ENGINE_PAGE for n in lengths.values())
    runner, w = build(dtype, num_blocks=pages, max_requests=3)
    cache = runner.cache
    rows = {rid: [] for rid in requests}
    seen = [set() for _ in cache.groups]
    reused = [False] * len(cache.groups)
    released_while_live = False
    for entries, ends in steps:
        batch = []
        for rid, start, count in entries:
            if not cache.has(rid):
                runner.begin(rid)
            batch.append(StepEntry(rid, requests[rid][start:start + count], list(range(count))))
        logits = runner.step(batch).cpu()
        at = 0
        for rid, start, count in entries:
            rows[rid].append(logits[at:at + count])
            at += count
        released_while_live = released_while_live or any(p < 0 for rid in cache.live_requests() for p in cache.page_list(2, rid))
        for rid in ends:
            for g in range(len(cache.groups)):
                held = {p for p in cache.page_list(g, rid) if p >= 0}
                reused[g] = reused[g] or bool(held & seen[g])
                seen[g] |= held
            runner.end(rid)
        cache.check_invariants()
    assert all(reused), f"groups whose pages no two requests used: {reused}"
    assert released_while_live, "the window never gave a page back while its request was live"
    for rid, tokens in requests.items():
        torch.testing.assert_close(torch.cat(rows[rid]), plain_logits(tokens, w), **TOL[dtype],
                                   msg=lambda m: f"{dtype} request {rid}: {m}")
    assert cache.free_pages() == [g.pool.num_pages for g in cache.groups]
