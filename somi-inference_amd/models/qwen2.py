"""The Qwen2.5 dense decoder as a plan.

Reference: somi_inference/models/qwen2.py:342-386 (embedding, identical pre-norm
layers of attention and SwiGLU, final RMSNorm) with tensor names as the
reference maps them from the checkpoint
(somi_inference/models/qwen2_adapter.py:149-190): ``model.embed_tokens.weight``,
``model.layers.{i}.input_layernorm/self_attn.{q,k,v,o}_proj/post_attention_layernorm/
mlp.{gate,up,down}_proj``, ``model.norm.weight``, ``lm_head.weight``.
"""

from __future__ import annotations

from ..config.qwen2 import Qwen2Config
from ..config.registry import register_architecture
from ..parts.base import PartSpec
from .plan import LayerSpec, ModelPlan


def qwen2_plan(config: Qwen2Config) -> ModelPlan:
    norm = PartSpec("rmsnorm", {"hidden_size": config.hidden_size, "eps": config.rms_norm_eps})
    feed_forward = PartSpec("swiglu", {"hidden_size": config.hidden_size,
                                       "intermediate_size": config.intermediate_size})
    position = PartSpec("rotary", {"head_dim": config.head_dim, "theta": config.rope_theta})
    layers = []
    for index in range(config.num_hidden_layers):
        mixer = PartSpec("gqa_attention", {
            "hidden_size": config.hidden_size,
            "num_heads": config.num_attention_heads,
            "num_kv_heads": config.num_key_value_heads,
            "head_dim": config.head_dim,
            "position": position,
            "qkv_bias": config.attention_bias,      # fixed on in the reference (qwen2.py:268-270)
            "out_bias": False,                      # fixed off in the reference (qwen2.py:271)
            "window": config.layer_window(index),
        })
        block = PartSpec("pre_norm", {"mixer": mixer, "feed_forward": feed_forward,
                                      "mixer_norm": norm, "ffn_norm": norm})
        layers.append(LayerSpec(f"model.layers.{index}", block))
    ignore = ["*rotary_emb.inv_freq"]               # computed buffer (qwen2_adapter.py:164-166)
    if config.tie_word_embeddings:
        ignore.append("lm_head.weight")             # a tied checkpoint may still carry it (qwen2_adapter.py:161-162)
    return ModelPlan(
        embedding=PartSpec("token_embedding", {"vocab_size": config.vocab_size, "hidden_size": config.hidden_size}),
        embedding_prefix="model.embed_tokens",
        layers=tuple(layers),
        final_norm=norm,
        final_norm_prefix="model.norm",
        head=PartSpec("lm_head", {"vocab_size": config.vocab_size, "hidden_size": config.hidden_size,
                                  "tied": config.tie_word_embeddings}),
        head_prefix="lm_head",
        ignore_weights=tuple(ignore),
        vocab_size=config.vocab_size,
        # the reference's rotary table has max_position_embeddings rows (qwen2_adapter.py:222, qwen2.py:72-81)
        max_positions=config.max_position_embeddings,
    )


register_architecture(Qwen2Config.architecture, Qwen2Config, qwen2_plan, replace=True)
