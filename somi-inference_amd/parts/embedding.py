"""Token embedding and LM head.

Reference: somi_inference/models/qwen2.py:360,382 (lookup) and
somi_inference/models/qwen2_adapter.py:60-62 (logits = h . E^T with the
embedding matrix, no bias).  The reference always ties the head; here a head
has a matrix of its own unless it is told to use the embedding's.
"""

from __future__ import annotations

import torch

from ..kernels import linear as linear_kernels
from ..kernels import ops
from ..weights.spec import MATRIX, WeightSpec
from .base import Fetch, Part, Runtime


class TokenEmbedding(Part):
    graph_safe = True

    def __init__(self, prefix: str, vocab_size: int, hidden_size: int) -> None:
        super().__init__(prefix)
        self.vocab_size, self.hidden_size = int(vocab_size), int(hidden_size)
        self.weight: torch.Tensor | None = None

    def weight_specs(self) -> list[WeightSpec]:
        return [WeightSpec(self.name("weight"), (self.vocab_size, self.hidden_size), MATRIX)]

    def load(self, fetch: Fetch, runtime: Runtime) -> None:
        super().load(fetch, runtime)
        self.weight = fetch(self.name("weight"))

    def forward(self, token_ids: torch.Tensor) -> torch.Tensor:
        """[N] int32 -> [N, H] float32 (the residual stream starts in float32)."""
        return ops.embedding(self.weight, token_ids)


class LMHead(Part):
    """logits = x . W^T in float32, for the rows that were asked for only."""
    graph_safe = True

    def __init__(self, prefix: str, vocab_size: int, hidden_size: int, tied: bool = False) -> None:
        super().__init__(prefix)
        self.vocab_size, self.hidden_size, self.tied = int(vocab_size), int(hidden_size), bool(tied)
        self.weight: torch.Tensor | None = None

    def weight_specs(self) -> list[WeightSpec]:
        if self.tied:
            return []
        return [WeightSpec(self.name("weight"), (self.vocab_size, self.hidden_size), MATRIX)]

    def load(self, fetch: Fetch, runtime: Runtime) -> None:
        super().load(fetch, runtime)
        if not self.tied:
            self.weight = fetch(self.name("weight"))

    def tie(self, embedding: TokenEmbedding) -> None:
        self.weight = embedding.weight

    def flops(self, tokens: int, attended: int = 0) -> float:
        """Of the logits of ``tokens`` rows."""
        return 2.0 * tokens * self.vocab_size * self.hidden_size

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return linear_kernels.linear(x, self.weight, None, torch.float32)
