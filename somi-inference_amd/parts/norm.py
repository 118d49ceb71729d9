"""RMSNorm.  Reference: somi_inference/models/qwen2.py:46-62."""

from __future__ import annotations

import torch

from ..kernels import ops
from ..weights.spec import VECTOR, Init, WeightSpec
from .base import Fetch, Norm, Runtime


class RMSNorm(Norm):
    """y = w * x * rsqrt(mean(x^2) + eps), no mean subtraction, no bias
    (qwen2.py:55-62).  Square, mean, rsqrt and scale are float32."""
    graph_safe = True
    fusable = True        # weight * (h / sqrt(mean(h^2) + eps)): what a projection can apply while it loads h

    def __init__(self, prefix: str, hidden_size: int, eps: float,
                 init: tuple[float, float] = (1.0, 0.1)) -> None:
        super().__init__(prefix)
        self.hidden_size = int(hidden_size)
        self.eps = float(eps)
        self._init = Init(*init)
        self.weight: torch.Tensor | None = None

    def weight_specs(self) -> list[WeightSpec]:
        return [WeightSpec(self.name("weight"), (self.hidden_size,), VECTOR, self._init)]

    def load(self, fetch: Fetch, runtime: Runtime) -> None:
        super().load(fetch, runtime)
        self.weight = fetch(self.name("weight"))

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return ops.rmsnorm(h, self.weight, self.eps, self.runtime.dtype)

    def add_forward(self, h: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
        return ops.rmsnorm(h, self.weight, self.eps, self.runtime.dtype, delta=delta)
