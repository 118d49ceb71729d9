"""A request as the scheduler tracks it.  Reference: ``Sequence`` / ``SequenceStatus``
(somi_inference/core/continuous_batching.py:13-34)."""

from __future__ import annotations

from dataclasses import dataclass, field
from enum import Enum
from typing import Hashable

from ..sampling.params import SamplingParams


class RequestStatus(Enum):
    WAITING = "waiting"
    RUNNING = "running"
    FINISHED = "finished"


@dataclass
class Request:
    request_id: Hashable
    prompt_tokens: list[int]
    max_new_tokens: int
    sampling_params: SamplingParams = field(default_factory=SamplingParams)
    seed: int = 0
    output_tokens: list[int] = field(default_factory=list)
    status: RequestStatus = RequestStatus.WAITING
    num_computed: int = 0            # tokens whose keys/values are in the cache
    num_preemptions: int = 0
    finish_reason: str | None = None

    def __post_init__(self) -> None:
        if self.max_new_tokens <= 0:            # asserted by the reference (continuous_batching.py:34)
            raise ValueError("max_new_tokens must be > 0")
        if len(self.prompt_tokens) < 1:
            raise ValueError("a request needs at least one prompt token")

    @property
    def all_tokens(self) -> list[int]:
        return self.prompt_tokens + self.output_tokens

    @property
    def num_pending(self) -> int:
        """Tokens not yet run: the rest of the prompt, or the one token sampled last."""
        return len(self.prompt_tokens) + len(self.output_tokens) - self.num_computed

    @property
    def max_cached_tokens(self) -> int:
        """Most tokens the request ever holds in the cache: the last sampled token is never
        run (continuous_batching.py:64-67)."""
        return len(self.prompt_tokens) + self.max_new_tokens - 1
