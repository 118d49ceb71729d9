"""A toy mixer with state of its own, defined here, is registered, built and stepped through the
engine's own runner and cache manager without a change to the package's files."""

from dataclasses import dataclass
from typing import ClassVar

import pytest
import torch

from somi_inference_amd.config import ModelConfig, config_from_dict, register_architecture, unregister_architecture
from somi_inference_amd.engine import StepEntry
from somi_inference_amd.models import LayerSpec, ModelPlan, make_runner, random_model
from somi_inference_amd.parts import FixedStateSpec, Mixer, PartSpec, register_part, unregister_part
from somi_inference_amd.weights import MATRIX, VECTOR, Init, WeightSpec

pytestmark = pytest.mark.gpu


class DecayMixer(Mixer):
    """y[t] = W . s[t],  s[t] = a * s[t-1] + x[t]  with a learned per-channel decay a in (0, 1):
    a running summary of fixed size per request, carried from portion to portion in a state slot."""

    def __init__(self, prefix, hidden_size):
        super().__init__(prefix)
        self.hidden_size = hidden_size

    def weight_specs(self):
        return [WeightSpec(self.name("decay"), (self.hidden_size,), VECTOR, Init(0.0, 1.0)),
                WeightSpec(self.name("out.weight"), (self.hidden_size, self.hidden_size), MATRIX, Init(0.0, 0.1))]

    def load(self, fetch, runtime):
        super().load(fetch, runtime)
        self.decay = torch.sigmoid(fetch(self.name("decay")))
        self.out = fetch(self.name("out.weight"))

    def cache_spec(self):
        return FixedStateSpec((self.hidden_size,), torch.float32)

    def forward(self, x, step, cache):
        out = torch.empty_like(x)
        for entry in step.entries:                       # tokens of one request in order, entries apart
            state = cache.state[entry.state_slot]
            for t in range(entry.start, entry.start + entry.length):
                state.mul_(self.decay).add_(x[t].float())
                out[t] = (self.out.float() @ state).to(x.dtype)
        return out


@dataclass(frozen=True)
class ToyConfig(ModelConfig):
    architecture: ClassVar[str] = "ToyDecayForCausalLM"
    vocab_size: int = 50
    hidden_size: int = 24
    layers: int = 3

    @classmethod
    def from_dict(cls, data):
        return cls(data["vocab_size"], data["hidden_size"], data["layers"])

    def to_dict(self):
        return {"architectures": [self.architecture], "vocab_size": self.vocab_size,
                "hidden_size": self.hidden_size, "layers": self.layers}


def toy_plan(config: ToyConfig) -> ModelPlan:
    norm = PartSpec("rmsnorm", {"hidden_size": config.hidden_size, "eps": 1e-6})
    decay = PartSpec("toy_decay", {"hidden_size": config.hidden_size})
    attention = PartSpec("gqa_attention", {"hidden_size": config.hidden_size, "num_heads": 2, "num_kv_heads": 1,
                                           "head_dim": 12, "position": PartSpec("rotary", {"head_dim": 12, "theta": 1e4})})
    ffn = PartSpec("swiglu", {"hidden_size": config.hidden_size, "intermediate_size": 40})
    layers = tuple(LayerSpec(f"model.layers.{i}", PartSpec("pre_norm", {
        "mixer": decay if i % 2 == 0 else attention, "feed_forward": ffn, "mixer_norm": norm, "ffn_norm": norm,
        "names": {"mixer": "mixer"}})) for i in range(config.layers))
    return ModelPlan(
        embedding=PartSpec("token_embedding", {"vocab_size": config.vocab_size, "hidden_size": config.hidden_size}),
        embedding_prefix="model.embed_tokens", layers=layers,
        final_norm=norm, final_norm_prefix="model.norm",
        head=PartSpec("lm_head", {"vocab_size": config.vocab_size, "hidden_size": config.hidden_size, "tied": True}),
        head_prefix="lm_head", vocab_size=config.vocab_size)


@pytest.fixture
def toy_registered():
    register_part("mixer", "toy_decay", DecayMixer)
    register_architecture(ToyConfig.architecture, ToyConfig, toy_plan)
    yield
    unregister_part("mixer", "toy_decay")
    unregister_architecture(ToyConfig.architecture)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_mixer_is_registered_built_and_stepped(toy_registered, dtype):
    arch, config = config_from_dict({"architectures": ["ToyDecayForCausalLM"], "vocab_size": 50, "hidden_size": 24, "layers": 3})
    assert isinstance(config, ToyConfig)
    model = random_model(config, seed=2, dtype=dtype)
    needs = model.cache_needs()
    assert isinstance(needs[0], FixedStateSpec) and isinstance(needs[2], FixedStateSpec)
    runner = make_runner(model, block_size=4, num_blocks=32, max_requests=3)
    assert runner.cache.layer_caches[0].state.shape == (3 + 1, 24)      # three requests and the padding slot
    gen = torch.Generator().manual_seed(0)
    a = torch.randint(0, 50, (23,), generator=gen).tolist()
    b = torch.randint(0, 50, (9,), generator=gen).tolist()

    def whole(tokens, rid):
        runner.begin(rid)
        out = runner.step([StepEntry(rid, tokens, list(range(len(tokens))))])
        runner.end(rid)
        return out
    want_a, want_b = whole(a, "a0"), whole(b, "b0")
    # now in portions, the two requests interleaved in shared batches: state must follow each request
    runner.begin("a")
    runner.begin("b")
    got_a = [runner.step([StepEntry("a", a[:5], list(range(5)))])]
    mixed = runner.step([StepEntry("a", a[5:12], list(range(7))), StepEntry("b", b[:4], list(range(4)))])
    got_a.append(mixed[:7])
    got_b = [mixed[7:]]
    mixed = runner.step([StepEntry("b", b[4:], list(range(5))), StepEntry("a", a[12:], list(range(11)))])
    got_b.append(mixed[:5])
    got_a.append(mixed[5:])
    tol = dict(atol=1e-5, rtol=1e-4) if dtype == "float32" else dict(atol=3e-2, rtol=3e-2)
    torch.testing.assert_close(torch.cat(got_a), want_a, **tol)
    torch.testing.assert_close(torch.cat(got_b), want_b, **tol)
    # a finished request's slot is used again and starts from zero
    runner.end("a")
    torch.testing.assert_close(whole(b, "b1"), want_b, **tol)
    runner.end("b")
    runner.cache.check_invariants()
