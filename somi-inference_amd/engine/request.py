"""A request as the scheduler tracks it.  Reference: ``Sequence`` / ``SequenceStatus``
(somi_inference/core/continuous_batching.py:13-34)."""

from __future__ import annotations

from collections.abc import Sequence
from dataclasses import dataclass, field
from enum import Enum
from itertools import chain, islice
from typing import Hashable

from ..sampling.params import SamplingParams


class RequestStatus(Enum):
    WAITING = "waiting"
    RUNNING = "running"
    FINISHED = "finished"


class TokenView(Sequence):
    """A request's prompt and output tokens as one sequence, without copying them (a request of thousands of tokens
    is looked at in every step)."""

    __slots__ = ("prompt", "output")

    def __init__(self, prompt: list[int], output: list[int]) -> None:
        self.prompt, self.output = prompt, output

    def __len__(self) -> int:
        return len(self.prompt) + len(self.output)

    def __iter__(self):
        return chain(self.prompt, self.output)

    def __getitem__(self, index):
        if isinstance(index, slice):
            start, stop, step = index.indices(len(self))
            if step != 1:
                return list(self)[index]
            split = len(self.prompt)
            if stop <= split:
                return self.prompt[start:stop]
            if start >= split:
                return self.output[start - split:stop - split]
            return self.prompt[start:] + self.output[:stop - split]
        if index < 0:
            index += len(self)
        split = len(self.prompt)
        return self.prompt[index] if index < split else self.output[index - split]

    def __eq__(self, other) -> bool:
        return len(self) == len(other) and all(a == b for a, b in zip(self, other))

    def __repr__(self) -> str:
        return f"TokenView({list(islice(self, 8))}{'...' if len(self) > 8 else ''}, {len(self)} tokens)"


@dataclass(eq=False)          # a request is itself: queues look it up by identity, not by comparing token lists
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
    def tokens(self) -> TokenView:
        """Prompt and output tokens as one sequence (a view, not a copy)."""
        return TokenView(self.prompt_tokens, self.output_tokens)

    @property
    def num_tokens(self) -> int:
        return len(self.prompt_tokens) + len(self.output_tokens)

    @property
    def num_pending(self) -> int:
        """Tokens not yet run: the rest of the prompt, or the one token sampled last."""
        return len(self.prompt_tokens) + len(self.output_tokens) - self.num_computed

    @property
    def max_cached_tokens(self) -> int:
        """Most tokens the request ever holds in the cache: the last sampled token is never
        run (continuous_batching.py:64-67)."""
        return len(self.prompt_tokens) + self.max_new_tokens - 1
