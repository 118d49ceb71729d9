"""Run-time options of the engine (not read from the model folder).

The reference takes these as keyword arguments of its entry point:
``num_blocks=256``, ``block_size=16``, ``max_concurrent=16``, ``dtype``
(somi_inference/entrypoints/llm.py:58-70, constants at :25-26).  The names and
defaults are kept; the token budget and the portion size are new, because the
reference runs whole prompts one at a time
(somi_inference/core/continuous_batching.py:200-203) and has no budget.
"""

from __future__ import annotations

from dataclasses import dataclass

from .base import ConfigError

DEFAULT_BLOCK_SIZE = 16
DEFAULT_NUM_BLOCKS = 256
DEFAULT_MAX_CONCURRENT = 16

_DTYPES = {"bfloat16": "bfloat16", "bf16": "bfloat16", "float32": "float32", "fp32": "float32"}


def normalize_dtype(name: object) -> str:
    """Accepts 'bfloat16'/'bf16'/'float32'/'fp32' or a torch dtype; returns the long name."""
    text = str(name).replace("torch.", "")
    if text not in _DTYPES:
        raise ConfigError(f"dtype must be one of bfloat16, float32; got {name!r}")
    return _DTYPES[text]


@dataclass(frozen=True)
class EngineConfig:
    dtype: str = "bfloat16"
    block_size: int = DEFAULT_BLOCK_SIZE        # tokens per cache page
    num_blocks: int = DEFAULT_NUM_BLOCKS        # pages per cache group
    max_concurrent: int = DEFAULT_MAX_CONCURRENT  # live requests
    max_num_batched_tokens: int = 2048          # token budget of one step
    max_chunk: int | None = None                # largest prompt portion; None = the budget
    device: str = "cuda:0"

    def __post_init__(self) -> None:
        object.__setattr__(self, "dtype", normalize_dtype(self.dtype))
        for key in ("block_size", "num_blocks", "max_concurrent", "max_num_batched_tokens"):
            if getattr(self, key) < 1:
                raise ConfigError(f"engine option '{key}' must be >= 1, got {getattr(self, key)}")
        if self.max_chunk is not None and self.max_chunk < 1:
            raise ConfigError(f"engine option 'max_chunk' must be >= 1, got {self.max_chunk}")

    @property
    def chunk(self) -> int:
        return min(self.max_chunk or self.max_num_batched_tokens, self.max_num_batched_tokens)
