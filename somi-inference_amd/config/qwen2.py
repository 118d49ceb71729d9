"""Typed configuration of the Qwen2.5 dense decoder.

Keys and defaults follow what the reference reads from the model's
config.json (somi_inference/models/qwen2_adapter.py:205-225): sizes, head
counts, ``rms_norm_eps``, ``max_position_embeddings`` and
``rope_parameters.rope_theta`` with 1e6 as the default.  The reference derives
``head_dim = hidden_size // num_attention_heads`` (qwen2_adapter.py:213) and
fixes q/k/v bias on, o bias off and SiLU in code (somi_inference/models/qwen2.py:
268-271, 223); here those are read when config.json carries them and default to
the reference's constants.  The reference always ties the LM head to the
embedding (qwen2_adapter.py:60-62, 161-162); ``tie_word_embeddings`` decides it
here, because the larger checkpoints of this architecture are untied.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, ClassVar

from .base import ConfigError, KeyReader, ModelConfig


@dataclass(frozen=True)
class Qwen2Config(ModelConfig):
    architecture: ClassVar[str] = "Qwen2ForCausalLM"

    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    head_dim: int
    rms_norm_eps: float = 1e-6
    rope_theta: float = 1_000_000.0
    max_position_embeddings: int = 32768
    tie_word_embeddings: bool = False
    attention_bias: bool = True
    hidden_act: str = "silu"
    use_sliding_window: bool = False
    sliding_window: int | None = None
    max_window_layers: int | None = None
    eos_token_id: int | None = None
    bos_token_id: int | None = None
    torch_dtype: str = "bfloat16"

    def __post_init__(self) -> None:
        for key in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                    "num_attention_heads", "num_key_value_heads", "head_dim",
                    "max_position_embeddings"):
            if getattr(self, key) < 1:
                raise ConfigError(f"config.json: '{key}' must be >= 1, got {getattr(self, key)}")
        # Grouped-query attention maps query head h to key/value head
        # h // (nq / nkv); the reference raises when this does not divide
        # (somi_inference/models/qwen2.py:116-123).
        if self.num_attention_heads % self.num_key_value_heads != 0:
            raise ConfigError(
                f"config.json: 'num_attention_heads' ({self.num_attention_heads}) must be "
                f"divisible by 'num_key_value_heads' ({self.num_key_value_heads})")
        # Rotate-half pairs element i with i + head_dim/2 (qwen2.py:95-99).
        if self.head_dim % 2 != 0:
            raise ConfigError(f"config.json: 'head_dim' must be even, got {self.head_dim}")
        if not self.rms_norm_eps >= 0.0:
            raise ConfigError(f"config.json: 'rms_norm_eps' must be >= 0, got {self.rms_norm_eps}")
        if not self.rope_theta > 0.0:
            raise ConfigError(f"config.json: 'rope_theta' must be > 0, got {self.rope_theta}")
        if self.hidden_act != "silu":
            raise ConfigError(
                f"config.json: 'hidden_act' is {self.hidden_act!r}; this architecture's "
                "feed-forward is SwiGLU and supports only 'silu'")
        if self.use_sliding_window:
            if self.sliding_window is None or self.sliding_window < 1:
                raise ConfigError(
                    "config.json: 'use_sliding_window' is true but 'sliding_window' is not a positive integer")
            if self.max_window_layers is None:
                raise ConfigError(
                    "config.json: 'use_sliding_window' is true but 'max_window_layers' is missing")

    # ------------------------------------------------------------------ reading
    @classmethod
    def from_dict(cls, data: dict[str, Any]) -> "Qwen2Config":
        r = KeyReader(data)
        hidden = r.integer("hidden_size", minimum=1)
        heads = r.integer("num_attention_heads", minimum=1)
        if r.has("head_dim"):
            head_dim = r.integer("head_dim", minimum=1)
        else:
            if hidden % heads != 0:
                raise ConfigError(
                    f"config.json: 'hidden_size' ({hidden}) is not divisible by "
                    f"'num_attention_heads' ({heads}) and no 'head_dim' is given")
            head_dim = hidden // heads
        # rope_theta lives under rope_parameters in newer exports
        # (qwen2_adapter.py:208-211) and at the top level in older ones.
        theta = 1_000_000.0
        params = r.sub("rope_parameters")
        if params is not None and params.has("rope_theta"):
            theta = params.number("rope_theta", positive=True)
            kind = params.raw("rope_type", "default")
            if kind not in ("default", None):
                raise ConfigError(f"config.json: rope_parameters.rope_type {kind!r} is not supported "
                                  "(the architecture uses unscaled rotary embeddings)")
        elif r.has("rope_theta"):
            theta = r.number("rope_theta", positive=True)
        if r.has("rope_scaling"):
            raise ConfigError("config.json: 'rope_scaling' is set; scaled rotary embeddings are not supported")
        eos = r.raw("eos_token_id", None)
        if isinstance(eos, list):
            eos = eos[0] if eos else None
        if eos is not None and (isinstance(eos, bool) or not isinstance(eos, int)):
            raise ConfigError(f"config.json: 'eos_token_id' must be an integer, got {eos!r}")
        return cls(
            vocab_size=r.integer("vocab_size", minimum=1),
            hidden_size=hidden,
            intermediate_size=r.integer("intermediate_size", minimum=1),
            num_hidden_layers=r.integer("num_hidden_layers", minimum=1),
            num_attention_heads=heads,
            num_key_value_heads=r.integer("num_key_value_heads", minimum=1),
            head_dim=head_dim,
            rms_norm_eps=r.number("rms_norm_eps", 1e-6),
            rope_theta=theta,
            max_position_embeddings=r.integer("max_position_embeddings", 32768, minimum=1),
            tie_word_embeddings=r.boolean("tie_word_embeddings", False),
            attention_bias=r.boolean("attention_bias", True),
            hidden_act=r.string("hidden_act", "silu"),
            use_sliding_window=r.boolean("use_sliding_window", False),
            sliding_window=r.optional_integer("sliding_window", minimum=1),
            max_window_layers=r.optional_integer("max_window_layers", minimum=0),
            eos_token_id=eos,
            bos_token_id=r.optional_integer("bos_token_id"),
            torch_dtype=r.string("torch_dtype", r.string("dtype", "bfloat16")),
        )

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {
            "architectures": [self.architecture],
            "model_type": "qwen2",
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "max_position_embeddings": self.max_position_embeddings,
            "tie_word_embeddings": self.tie_word_embeddings,
            "attention_bias": self.attention_bias,
            "hidden_act": self.hidden_act,
            "use_sliding_window": self.use_sliding_window,
            "torch_dtype": self.torch_dtype,
        }
        for key in ("sliding_window", "max_window_layers", "eos_token_id", "bos_token_id"):
            if getattr(self, key) is not None:
                out[key] = getattr(self, key)
        return out

    # ------------------------------------------------------------ derived facts
    def layer_window(self, layer: int) -> int | None:
        """How many keys (itself included) a token of ``layer`` attends to; None = all.

        The reference stores a ``sliding_window_size`` on its attention module
        and never reads it (somi_inference/models/qwen2.py:262, 272), so its
        attention is always over all keys.  Here the config.json keys keep
        their meaning: with ``use_sliding_window``, layers from
        ``max_window_layers`` on see the last ``sliding_window`` keys only.
        """
        if not self.use_sliding_window:
            return None
        assert self.max_window_layers is not None
        return self.sliding_window if layer >= self.max_window_layers else None
