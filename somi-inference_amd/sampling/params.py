"""Per-request sampling options.  Reference: ``SamplingParams`` (somi_inference/core/sampler.py:11-25)."""

from __future__ import annotations

from dataclasses import dataclass


@dataclass(frozen=True)
class SamplingParams:
    """Names, defaults and ranges are the reference's (sampler.py:15-25); ``seed`` is new:
    the reference draws from torch's global generator, here every request has its own
    counter-based stream so its tokens do not depend on what else is in the batch."""

    temperature: float = 1.0          # 0.0 = greedy; top-k and top-p are then skipped
    top_k: int = -1                   # -1 = off
    top_p: float = 1.0                # 1.0 = off
    repetition_penalty: float = 1.0   # 1.0 = off
    seed: int | None = None           # None = derived from the engine's seed and the request's number

    def __post_init__(self) -> None:
        if not self.temperature >= 0.0:
            raise ValueError("temperature must be >= 0.0")
        if not (self.top_k == -1 or self.top_k > 0):
            raise ValueError("top_k must be -1 or > 0")
        if not 0.0 < self.top_p <= 1.0:
            raise ValueError("top_p must be in (0.0, 1.0]")
        if not self.repetition_penalty > 0.0:
            raise ValueError("repetition_penalty must be > 0.0")
