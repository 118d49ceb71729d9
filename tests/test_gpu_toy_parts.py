"""Toy parts defined here (a feed-forward with routing, two position encodings, another block arrangement)
and a run that reads an earlier run's cache are registered, built and stepped through the engine's own
runner and cache manager without a change to the package's files.  Each model is compared with a plain
computation written here, whole and in portions."""

import math

import pytest
import torch

from plain import qwen2_plain as plain
from somi_inference_amd.cache import CacheManager
from somi_inference_amd.engine import ModelRunner, StepEntry
from somi_inference_amd.models import DecoderModel, LayerSpec, ModelPlan
from somi_inference_amd.parts import (Block, FeedForward, PartSpec, PositionEncoding, Runtime, build_part,
                                      register_part, unregister_part)
from somi_inference_amd.weights import MATRIX, Init, RandomSource, WeightSpec

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": dict(atol=3e-5, rtol=1e-4), "bfloat16": dict(atol=4e-2, rtol=4e-2)}
HIDDEN, VOCAB, EPS = 48, 61, 1e-6


# ------------------------------------------------------------------------------------------ toy parts
class Top1Experts(FeedForward):
    """Routing: float32 router logits, the best expert per token, its output scaled by its softmax weight."""

    def __init__(self, prefix, hidden_size, intermediate_size, num_experts):
        super().__init__(prefix)
        self.hidden_size, self.intermediate_size, self.num_experts = hidden_size, intermediate_size, num_experts

    def weight_specs(self):
        specs = [WeightSpec(self.name("router.weight"), (self.num_experts, self.hidden_size), MATRIX, Init(0.0, 0.5))]
        for e in range(self.num_experts):
            specs += [WeightSpec(self.name(f"experts.{e}.up.weight"), (self.intermediate_size, self.hidden_size), MATRIX, Init(0.0, 0.2)),
                      WeightSpec(self.name(f"experts.{e}.down.weight"), (self.hidden_size, self.intermediate_size), MATRIX, Init(0.0, 0.2))]
        return specs

    def load(self, fetch, runtime):
        super().load(fetch, runtime)
        self.router = fetch(self.name("router.weight")).float()
        self.up = [fetch(self.name(f"experts.{e}.up.weight")) for e in range(self.num_experts)]
        self.down = [fetch(self.name(f"experts.{e}.down.weight")) for e in range(self.num_experts)]

    def forward(self, x, step=None):
        gates = torch.softmax(x.float() @ self.router.t(), dim=-1)
        weight, choice = gates.max(dim=-1)
        out = torch.zeros_like(x)
        for e in range(self.num_experts):
            rows = (choice == e).nonzero().flatten()
            if rows.numel():
                hidden = torch.relu(x[rows] @ self.up[e].t())
                out[rows] = ((hidden @ self.down[e].t()).float() * weight[rows, None]).to(x.dtype)
        return out


class TwoChannelRotation(PositionEncoding):
    """A rotation of its own, through the hook for encodings that offer no table: channels 0 and 1 of every
    q and k head are turned by the angle position * rate."""

    def __init__(self, prefix, rate):
        super().__init__(prefix)
        self.rate = rate

    def encode_qk(self, qkv, step, nq, nkv, head_dim):
        heads = qkv[:, :(nq + nkv) * head_dim].view(qkv.shape[0], nq + nkv, head_dim)
        angle = step.positions.float() * self.rate
        cos, sin = torch.cos(angle)[:, None], torch.sin(angle)[:, None]
        a, b = heads[..., 0].float(), heads[..., 1].float()
        turned = (a * cos - b * sin).to(qkv.dtype), (a * sin + b * cos).to(qkv.dtype)    # both before either is written
        heads[..., 0], heads[..., 1] = turned


class LearnedPositions(PositionEncoding):
    """A learned vector per absolute position, added to the embedded tokens."""

    def __init__(self, prefix, hidden_size, max_positions):
        super().__init__(prefix)
        self.hidden_size, self.max_positions = hidden_size, max_positions

    def weight_specs(self):
        return [WeightSpec(self.name("weight"), (self.max_positions, self.hidden_size), MATRIX, Init(0.0, 0.5))]

    def load(self, fetch, runtime):
        super().load(fetch, runtime)
        self.table = fetch(self.name("weight")).float()

    def encode_embeddings(self, h, step):
        h += self.table[step.positions.long()]


class ParallelBlock(Block):
    """h += mixer(norm(h)) + feed_forward(norm(h)): one norm, both sub-layers read the same rows."""

    def __init__(self, prefix, mixer, feed_forward, norm):
        super().__init__(prefix)
        self.norm = build_part("norm", norm, prefix=self.name("norm"))
        self.mixer = build_part("mixer", mixer, prefix=self.name("self_attn"))
        self.feed_forward = build_part("feed_forward", feed_forward, prefix=self.name("mlp"))

    def parts(self):
        return [self.norm, self.mixer, self.feed_forward]

    def forward(self, stream, step, cache):
        x = stream.normed(self.norm)
        stream.add(self.mixer.forward(x, step, cache))
        stream.add(self.feed_forward.forward(x, step))


@pytest.fixture
def toys():
    register_part("feed_forward", "toy_top1_experts", Top1Experts)
    register_part("position", "toy_two_channel_rotation", TwoChannelRotation)
    register_part("position", "toy_learned_positions", LearnedPositions)
    register_part("block", "toy_parallel", ParallelBlock)
    yield
    unregister_part("feed_forward", "toy_top1_experts")
    unregister_part("position", "toy_two_channel_rotation")
    unregister_part("position", "toy_learned_positions")
    unregister_part("block", "toy_parallel")


# ---------------------------------------------------------------------------------------------- helpers
NORM = PartSpec("rmsnorm", {"hidden_size": HIDDEN, "eps": EPS})
ROTARY = PartSpec("rotary", {"head_dim": 16, "theta": 1e4})
SWIGLU = PartSpec("swiglu", {"hidden_size": HIDDEN, "intermediate_size": 80})


def attention(position=ROTARY, **more):
    return PartSpec("gqa_attention", {"hidden_size": HIDDEN, "num_heads": 4, "num_kv_heads": 2, "head_dim": 16,
                                      "position": position, **more})


def pre_norm(index, mixer, feed_forward=SWIGLU):
    return LayerSpec(f"model.layers.{index}", PartSpec("pre_norm", {"mixer": mixer, "feed_forward": feed_forward,
                                                                     "mixer_norm": NORM, "ffn_norm": NORM}))


def plan_of(layers, **more):
    return ModelPlan(embedding=PartSpec("token_embedding", {"vocab_size": VOCAB, "hidden_size": HIDDEN}),
                     embedding_prefix="model.embed_tokens", layers=tuple(layers), final_norm=NORM,
                     final_norm_prefix="model.norm",
                     head=PartSpec("lm_head", {"vocab_size": VOCAB, "hidden_size": HIDDEN, "tied": True}),
                     head_prefix="lm_head", vocab_size=VOCAB, **more)


def build(plan, dtype, seed=5):
    """The model with seeded random weights (projections enlarged so that attention is not flat), its runner,
    and the weights as float32 CPU tensors for the plain side."""
    model = DecoderModel(plan, Runtime(DT[dtype], DEV))
    kept = {}

    class Keeping(RandomSource):
        def read(self, name, device):
            tensor = super().read(name, device)
            if "_proj.weight" in name:
                tensor = (tensor.float() * 6.0).to(tensor.dtype)
            kept[name] = tensor.float().cpu()
            return tensor
    model.load(Keeping(model.weight_specs(), seed))
    cache = CacheManager(model.cache_needs(), block_size=8, num_blocks=24, max_requests=2, dtype=DT[dtype], device=DEV)
    return ModelRunner(model, cache), kept


def run_whole_and_in_portions(runner, tokens, want, dtype):
    for sizes in ([len(tokens)], [3, 11, 2, len(tokens) - 16]):
        runner.begin("r")
        outs, at = [], 0
        for size in sizes:
            outs.append(runner.step([StepEntry("r", tokens[at:at + size], list(range(size)))]))
            at += size
        runner.end("r")
        torch.testing.assert_close(torch.cat(outs).cpu(), want, **TOL[dtype])
    runner.cache.check_invariants()


def plain_qkv(x, w, prefix, positions, rotate):
    """q, k, v heads ([heads, T, 16]) of the toy attention from normed rows x, q and k turned by ``rotate``."""
    t = x.shape[0]
    q = plain.linear(x, w[f"{prefix}.q_proj.weight"], w[f"{prefix}.q_proj.bias"]).view(t, 4, 16).transpose(0, 1)
    out = [rotate(q, positions)]
    if f"{prefix}.k_proj.weight" in w:
        k = plain.linear(x, w[f"{prefix}.k_proj.weight"], w[f"{prefix}.k_proj.bias"]).view(t, 2, 16).transpose(0, 1)
        v = plain.linear(x, w[f"{prefix}.v_proj.weight"], w[f"{prefix}.v_proj.bias"]).view(t, 2, 16).transpose(0, 1)
        out += [rotate(k, positions), v]
    return out


def plain_attend(q, k, v, w, prefix):
    t = q.shape[1]
    attended = plain.causal_attention(q, k, v)                  # [4, T, 16], query head h reads kv head h // 2
    return plain.linear(attended.transpose(0, 1).reshape(t, 64), w[f"{prefix}.o_proj.weight"])


def rope(heads, positions):
    cos, sin = plain.rope_cos_sin(positions, 16, 1e4)
    return plain.apply_rope(heads, cos, sin)


def plain_ffn(x, w, prefix):
    return plain.swiglu(x, w[f"{prefix}.gate_proj.weight"], w[f"{prefix}.up_proj.weight"], w[f"{prefix}.down_proj.weight"])


def plain_logits(h, w):
    return plain.rms_norm(h, w["model.norm.weight"], EPS) @ w["model.embed_tokens.weight"].t()


def tokens_of(n, seed=1):
    return torch.randint(0, VOCAB, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


# ------------------------------------------------------------------------------------------------ tests
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_run_may_read_the_cache_an_earlier_run_wrote(dtype):
    """Layer 1 has no k/v projections: its queries attend over the keys and values that layer 0 wrote
    (``cache_from``); layer 2 has a cache of its own again."""
    plan = plan_of([pre_norm(0, attention()), pre_norm(1, attention(shares_cache=True)), pre_norm(2, attention())],
                   cache_from={1: 0})
    runner, w = build(plan, dtype)
    assert "model.layers.1.self_attn.k_proj.weight" not in w
    needs = runner.model.cache_needs()
    assert needs[1] == 0 and runner.cache.layer_caches[1].k is runner.cache.layer_caches[0].k
    assert runner.cache.layer_caches[1].writes is False and runner.cache.layer_caches[2].k is not runner.cache.layer_caches[0].k
    tokens, positions = tokens_of(29), torch.arange(29)
    h = w["model.embed_tokens.weight"][torch.tensor(tokens)]
    shared = None
    for index in range(3):
        p = f"model.layers.{index}"
        heads = plain_qkv(plain.rms_norm(h, w[f"{p}.input_layernorm.weight"], EPS), w, f"{p}.self_attn", positions, rope)
        if index == 0:
            shared = heads[1:]
        q, (k, v) = heads[0], (shared if index == 1 else heads[1:])
        h = h + plain_attend(q, k, v, w, f"{p}.self_attn")
        h = h + plain_ffn(plain.rms_norm(h, w[f"{p}.post_attention_layernorm.weight"], EPS), w, f"{p}.mlp")
    run_whole_and_in_portions(runner, tokens, plain_logits(h, w), dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_feed_forward_with_routing(toys, dtype):
    experts = PartSpec("toy_top1_experts", {"hidden_size": HIDDEN, "intermediate_size": 40, "num_experts": 3})
    plan = plan_of([pre_norm(0, attention(), experts), pre_norm(1, attention())])
    runner, w = build(plan, dtype)
    tokens, positions = tokens_of(29), torch.arange(29)
    h = w["model.embed_tokens.weight"][torch.tensor(tokens)]
    used = set()
    for index in range(2):
        p = f"model.layers.{index}"
        q, k, v = plain_qkv(plain.rms_norm(h, w[f"{p}.input_layernorm.weight"], EPS), w, f"{p}.self_attn", positions, rope)
        h = h + plain_attend(q, k, v, w, f"{p}.self_attn")
        x = plain.rms_norm(h, w[f"{p}.post_attention_layernorm.weight"], EPS)
        if index == 1:
            h = h + plain_ffn(x, w, f"{p}.mlp")
            continue
        gates = torch.softmax(x @ w[f"{p}.mlp.router.weight"].t(), dim=-1)
        weight, choice = gates.max(dim=-1)
        top2 = gates.topk(2, dim=-1).values
        assert float((top2[:, 0] - top2[:, 1]).min()) > 0.02, "a routing decision too close to call for bfloat16"
        out = torch.zeros_like(x)
        for row in range(29):
            e = int(choice[row])
            used.add(e)
            hidden = torch.relu(x[row] @ w[f"{p}.mlp.experts.{e}.up.weight"].t())
            out[row] = (hidden @ w[f"{p}.mlp.experts.{e}.down.weight"].t()) * weight[row]
        h = h + out
    assert len(used) >= 2
    run_whole_and_in_portions(runner, tokens, plain_logits(h, w), dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_position_encodings_through_both_hooks(toys, dtype):
    """Layer 0 turns two channels of q and k itself (no table for the fused kernel); learned absolute positions
    are added to the embedded tokens; layer 1 has no position encoding at all."""
    rate = 0.37
    plan = plan_of([pre_norm(0, attention(PartSpec("toy_two_channel_rotation", {"rate": rate}))),
                    pre_norm(1, attention(PartSpec("none", {})))],
                   embedding_position=PartSpec("toy_learned_positions", {"hidden_size": HIDDEN, "max_positions": 40}),
                   embedding_position_prefix="model.positions")
    runner, w = build(plan, dtype)
    assert runner.decode_graphs is False                       # toy parts do not claim to be safe to capture
    tokens, positions = tokens_of(29), torch.arange(29)

    def two_channels(heads, pos):
        angle = pos.float() * rate
        cos, sin = torch.cos(angle)[None, :], torch.sin(angle)[None, :]
        out = heads.clone()
        out[..., 0] = heads[..., 0] * cos - heads[..., 1] * sin
        out[..., 1] = heads[..., 0] * sin + heads[..., 1] * cos
        return out
    h = w["model.embed_tokens.weight"][torch.tensor(tokens)] + w["model.positions.weight"][positions]
    for index, rotate in enumerate([two_channels, lambda heads, pos: heads]):
        p = f"model.layers.{index}"
        q, k, v = plain_qkv(plain.rms_norm(h, w[f"{p}.input_layernorm.weight"], EPS), w, f"{p}.self_attn", positions, rotate)
        h = h + plain_attend(q, k, v, w, f"{p}.self_attn")
        h = h + plain_ffn(plain.rms_norm(h, w[f"{p}.post_attention_layernorm.weight"], EPS), w, f"{p}.mlp")
    run_whole_and_in_portions(runner, tokens, plain_logits(h, w), dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_block_arrangement(toys, dtype):
    parallel = LayerSpec("model.layers.0", PartSpec("toy_parallel", {"mixer": attention(), "feed_forward": SWIGLU, "norm": NORM}))
    plan = plan_of([parallel, pre_norm(1, attention())])
    runner, w = build(plan, dtype)
    tokens, positions = tokens_of(29), torch.arange(29)
    h = w["model.embed_tokens.weight"][torch.tensor(tokens)]
    x = plain.rms_norm(h, w["model.layers.0.norm.weight"], EPS)
    q, k, v = plain_qkv(x, w, "model.layers.0.self_attn", positions, rope)
    h = h + plain_attend(q, k, v, w, "model.layers.0.self_attn") + plain_ffn(x, w, "model.layers.0.mlp")
    p = "model.layers.1"
    q, k, v = plain_qkv(plain.rms_norm(h, w[f"{p}.input_layernorm.weight"], EPS), w, f"{p}.self_attn", positions, rope)
    h = h + plain_attend(q, k, v, w, f"{p}.self_attn")
    h = h + plain_ffn(plain.rms_norm(h, w[f"{p}.post_attention_layernorm.weight"], EPS), w, f"{p}.mlp")
    run_whole_and_in_portions(runner, tokens, plain_logits(h, w), dtype)
    assert math.isfinite(float(plain_logits(h, w).abs().max()))
