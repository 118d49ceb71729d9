"""Dense SwiGLU feed-forward.  Reference: somi_inference/models/qwen2.py:209-229."""

from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.spec import MATRIX, WeightSpec
from .base import FeedForward, Fetch, Runtime
from .linear import Projection


class SwiGLU(FeedForward):
    """y = down(silu(gate(x)) * up(x)), no biases.  gate and up are stacked into one
    ``[2I, H]`` matrix, gate rows first, as the reference merges them at load
    (somi_inference/models/qwen2_adapter.py:183-190, 244-248; qwen2.py:228 chunks the result)."""
    graph_safe = True

    def __init__(self, prefix: str, hidden_size: int, intermediate_size: int) -> None:
        super().__init__(prefix)
        self.hidden_size, self.intermediate_size = int(hidden_size), int(intermediate_size)

    def weight_specs(self) -> list[WeightSpec]:
        h, i = self.hidden_size, self.intermediate_size
        return [WeightSpec(self.name("gate_proj.weight"), (i, h), MATRIX),
                WeightSpec(self.name("up_proj.weight"), (i, h), MATRIX),
                WeightSpec(self.name("down_proj.weight"), (h, i), MATRIX)]

    def load(self, fetch: Fetch, runtime: Runtime) -> None:
        super().load(fetch, runtime)
        self.gate_up = Projection.stacked([fetch(self.name("gate_proj.weight")), fetch(self.name("up_proj.weight"))])
        self.down = Projection(fetch(self.name("down_proj.weight")))

    def forward(self, x: torch.Tensor, step=None) -> torch.Tensor:
        return self.down(ops.silu_mul(self.gate_up(x)))
