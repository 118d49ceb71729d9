"""Typed configuration, architecture registry and engine options (no GPU)."""

import json

import pytest

from somi_inference_amd.config import (ConfigError, EngineConfig, Qwen2Config, config_from_dict,
                                       read_config_json, register_architecture, registered_architectures,
                                       resolve_architecture, unregister_architecture)
from somi_inference_amd.models import collect_weight_specs, qwen2_plan

BASE = dict(architectures=["Qwen2ForCausalLM"], model_type="qwen2", vocab_size=503, hidden_size=192,
            intermediate_size=512, num_hidden_layers=3, num_attention_heads=6, num_key_value_heads=1)


def test_reads_the_architectures_own_keys_with_reference_defaults():
    arch, cfg = config_from_dict(dict(BASE))
    assert arch.name == "Qwen2ForCausalLM" and isinstance(cfg, Qwen2Config)
    assert cfg.head_dim == 32                      # hidden // heads (reference: qwen2_adapter.py:213)
    assert cfg.rms_norm_eps == 1e-6 and cfg.rope_theta == 1_000_000.0
    assert cfg.tie_word_embeddings is False and cfg.attention_bias is True and cfg.hidden_act == "silu"


def test_rope_theta_from_rope_parameters_or_top_level():
    assert config_from_dict(dict(BASE, rope_parameters={"rope_theta": 12345.0}))[1].rope_theta == 12345.0
    assert config_from_dict(dict(BASE, rope_theta=777.0))[1].rope_theta == 777.0


def test_explicit_head_dim_wins_over_the_quotient():
    assert config_from_dict(dict(BASE, head_dim=48))[1].head_dim == 48


@pytest.mark.parametrize("change, word", [
    (dict(vocab_size=None), "vocab_size"),
    (dict(hidden_size="192"), "hidden_size"),
    (dict(num_attention_heads=5), "divisible"),
    (dict(num_key_value_heads=4), "divisible"),
    (dict(head_dim=31), "even"),
    (dict(hidden_act="gelu"), "silu"),
    (dict(rope_scaling={"type": "yarn", "factor": 4.0}), "rope_scaling"),
    (dict(use_sliding_window=True), "sliding_window"),
    (dict(rms_norm_eps=-1.0), "rms_norm_eps"),
    (dict(num_hidden_layers=0), "num_hidden_layers"),
    (dict(tie_word_embeddings="yes"), "tie_word_embeddings"),
])
def test_each_violated_rule_names_its_key(change, word):
    data = dict(BASE)
    data.update(change)
    if change.get("vocab_size", 1) is None:
        del data["vocab_size"]
    with pytest.raises(ConfigError, match=word):
        config_from_dict(data)


def test_to_dict_round_trips():
    cfg = config_from_dict(dict(BASE, use_sliding_window=True, sliding_window=20, max_window_layers=1,
                                eos_token_id=7, tie_word_embeddings=True))[1]
    again = config_from_dict(json.loads(json.dumps(cfg.to_dict())))[1]
    assert again == cfg
    assert [cfg.layer_window(i) for i in range(3)] == [None, 20, 20]


def test_unknown_architecture_lists_the_registered_ones():
    # the reference: ValueError("Unsupported model type: X") (models/loader.py:24-26)
    with pytest.raises(ConfigError, match="Unsupported architecture.*Qwen2ForCausalLM"):
        config_from_dict(dict(BASE, architectures=["LlamaForCausalLM"]))
    with pytest.raises(ConfigError, match="architectures"):
        config_from_dict({k: v for k, v in BASE.items() if k != "architectures"})


def test_registry_takes_a_new_architecture_without_touching_the_package():
    class ToyConfig(Qwen2Config):
        architecture = "ToyForCausalLM"
    register_architecture("ToyForCausalLM", ToyConfig, qwen2_plan)
    try:
        assert "ToyForCausalLM" in registered_architectures()
        assert resolve_architecture("ToyForCausalLM").config_class is ToyConfig
        with pytest.raises(ConfigError, match="already registered"):
            register_architecture("ToyForCausalLM", ToyConfig, qwen2_plan)
    finally:
        unregister_architecture("ToyForCausalLM")


def test_read_config_json_errors_name_the_file(tmp_path):
    with pytest.raises(ConfigError, match="config.json"):
        read_config_json(tmp_path)
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError, match="not valid JSON"):
        read_config_json(tmp_path)


def test_plan_has_no_size_of_its_own():
    """Every size in the plan comes from the configuration: two configurations, two sets of shapes."""
    cfg = config_from_dict(dict(BASE, tie_word_embeddings=False))[1]
    shapes = {s.name: s.shape for s in collect_weight_specs(qwen2_plan(cfg))}
    assert shapes["model.embed_tokens.weight"] == (503, 192)
    assert shapes["model.layers.2.self_attn.q_proj.weight"] == (6 * 32, 192)
    assert shapes["model.layers.0.self_attn.k_proj.bias"] == (32,)
    assert shapes["model.layers.1.mlp.gate_proj.weight"] == (512, 192)
    assert shapes["lm_head.weight"] == (503, 192)
    assert "model.layers.0.self_attn.o_proj.bias" not in shapes     # o has no bias (reference qwen2.py:271)
    tied = config_from_dict(dict(BASE, tie_word_embeddings=True))[1]
    assert "lm_head.weight" not in {s.name for s in collect_weight_specs(qwen2_plan(tied))}
    no_bias = config_from_dict(dict(BASE, attention_bias=False))[1]
    assert not any(s.name.endswith(".bias") for s in collect_weight_specs(qwen2_plan(no_bias)))


def test_engine_options_keep_the_reference_names_and_defaults():
    opts = EngineConfig()
    assert (opts.num_blocks, opts.block_size, opts.max_concurrent) == (256, 16, 16)   # entrypoints/llm.py:25-26, 62-64
    assert EngineConfig(dtype="fp32").dtype == "float32" and EngineConfig(dtype="torch.bfloat16".replace("torch.", "")).dtype == "bfloat16"
    assert EngineConfig(max_num_batched_tokens=100, max_chunk=512).chunk == 100
    with pytest.raises(ConfigError):
        EngineConfig(dtype="float16")
    with pytest.raises(ConfigError):
        EngineConfig(block_size=0)
